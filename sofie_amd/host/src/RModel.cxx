// RModel: tensor registries, operator list, memory plan and Session emission for the HIP path.
// Structure of the generated Session follows the reference's emitter
// (src/SOFIE_core/src/RModel.cxx:574-910): tensor members, intermediate pool with offsets,
// constructor that reads the text weight file with name/length checks, infer() that runs every
// operator's Generate() text and returns a std::vector copy of the output.
#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator_BatchNormalization.hxx"
#include "SOFIE/ROperator_Conv.hxx"
#include "SOFIE/ROperator_Gemm.hxx"
#include "SOFIE/ROperator_Pool.hxx"
#include "SOFIE/ROperator_Quantized.hxx"

#include <cmath>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <limits>

namespace SOFIE {

std::underlying_type_t<Options> operator|(Options opA, Options opB)
{
   return static_cast<std::underlying_type_t<Options>>(opA) | static_cast<std::underlying_type_t<Options>>(opB);
}
std::underlying_type_t<Options> operator|(std::underlying_type_t<Options> opA, Options opB)
{
   return opA | static_cast<std::underlying_type_t<Options>>(opB);
}

RModel::RModel(std::string name, std::string parsedtime) : fFileName(name), fParseTime(parsedtime)
{
   // model name = file name without directory and extension, as the reference derives it
   fName = fFileName.substr(0, fFileName.rfind("."));
   fName = UTILITY::Clean_name(fName.substr(fName.find_last_of("/\\") + 1));
}

const std::vector<size_t> &RModel::GetTensorShape(std::string name) const
{
   auto f = fReadyInputTensorInfos.find(name);
   if (f != fReadyInputTensorInfos.end()) return f->second.shape;
   auto f2 = fInitializedTensors.find(name);
   if (f2 != fInitializedTensors.end()) return f2->second.shape();
   auto f4 = fIntermediateTensorInfos.find(name);
   if (f4 != fIntermediateTensorInfos.end()) return f4->second.shape;
   throw std::runtime_error("TMVA SOFIE tensor [" + name + "] for which the shape is requested is not found");
}

std::vector<Dim> RModel::GetDynamicTensorShape(std::string name) const
{
   return ConvertShapeToDim(GetTensorShape(name));
}

const ETensorType &RModel::GetTensorType(std::string name) const
{
   auto f = fReadyInputTensorInfos.find(name);
   if (f != fReadyInputTensorInfos.end()) return f->second.type;
   auto f2 = fInitializedTensors.find(name);
   if (f2 != fInitializedTensors.end()) return f2->second.type();
   auto f4 = fIntermediateTensorInfos.find(name);
   if (f4 != fIntermediateTensorInfos.end()) return f4->second.type;
   throw std::runtime_error("TMVA SOFIE tensor [" + name + "] for which the type is requested is not found, model name: " +
                            fName);
}

bool RModel::CheckIfTensorAlreadyExist(std::string tensor_name)
{
   return fReadyInputTensorInfos.count(tensor_name) || fInitializedTensors.count(tensor_name) ||
          fIntermediateTensorInfos.count(tensor_name);
}

bool RModel::IsInitializedTensor(const std::string &name) const { return fInitializedTensors.count(name) != 0; }
bool RModel::IsReadyInputTensor(const std::string &name) const { return fReadyInputTensorInfos.count(name) != 0; }

void RModel::AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<Dim> shape)
{
   std::vector<size_t> s = ConvertShapeToInt(shape);
   if (s.empty() && !shape.empty()) {
      // a parametric shape (a named batch dimension): kept until Initialize is told the value, as in the
      // reference (RModel_Base / RModel.cxx:398-463)
      input_name = UTILITY::Clean_name(input_name);
      if (CheckIfTensorAlreadyExist(input_name))
         throw std::runtime_error("TMVA-SOFIE: input tensor with name " + input_name + " already exists \n");
      fInputTensorInfos[input_name] = ParametricInput{type, shape};
      return;
   }
   AddInputTensorInfo(input_name, type, s);
}

void RModel::AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<size_t> shape)
{
   input_name = UTILITY::Clean_name(input_name);
   if (CheckIfTensorAlreadyExist(input_name))
      throw std::runtime_error("TMVA-SOFIE: input tensor with name " + input_name + " already exists \n");
   fReadyInputTensorInfos[input_name] = TensorInfo{type, shape};
}

void RModel::AddInputTensorName(std::string input_name) { fInputTensorNames.emplace_back(UTILITY::Clean_name(input_name)); }

void RModel::AddOperator(std::unique_ptr<ROperator> op, int order_execution)
{
   AddBlasRoutines(op->GetBlasRoutines());
   for (auto &stdlib : op->GetStdLibs()) AddNeededStdLib(stdlib);
   if (order_execution >= 0 && order_execution <= (int)fOperators.size())
      fOperators.insert(fOperators.begin() + order_execution, std::move(op));
   else
      fOperators.push_back(std::move(op));
}

void RModel::AddInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape,
                                  std::shared_ptr<void> data)
{
   tensor_name = UTILITY::Clean_name(tensor_name);
   if (CheckIfTensorAlreadyExist(tensor_name))
      throw std::runtime_error("TMVA-SOFIE: initialized tensor with name " + tensor_name + " already exists \n");
   fInitializedTensors[tensor_name] = InitializedTensor{type, shape, data};
}

void RModel::UpdateInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape,
                                     std::shared_ptr<void> data)
{
   tensor_name = UTILITY::Clean_name(tensor_name);
   if (!fInitializedTensors.count(tensor_name))
      throw std::runtime_error("TMVA-SOFIE: tensor " + tensor_name + " not found when trying to update it");
   fInitializedTensors[tensor_name] = InitializedTensor{type, shape, data};
}

std::shared_ptr<void> RModel::GetInitializedTensorData(std::string tensor_name)
{
   auto f = fInitializedTensors.find(tensor_name);
   if (f == fInitializedTensors.end())
      throw std::runtime_error("TMVA-SOFIE: tensor " + tensor_name + " not found when trying to get its data");
   return f->second.sharedptr();
}

void RModel::SetNotWritableInitializedTensor(const std::string &tensor_name)
{
   auto f = fInitializedTensors.find(tensor_name);
   if (f == fInitializedTensors.end())
      throw std::runtime_error("TMVA-SOFIE: initialized tensor " + tensor_name + " not found");
   f->second.SetNotWritable();
}

void RModel::AddIntermediateTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape)
{
   tensor_name = UTILITY::Clean_name(tensor_name);
   if (CheckIfTensorAlreadyExist(tensor_name))
      throw std::runtime_error("TMVA-SOFIE: intermediate tensor with name " + tensor_name + " already exists \n");
   fIntermediateTensorInfos[tensor_name] = TensorInfo{type, shape};
}

void RModel::AddIntermediateTensor(std::string tensor_name, ETensorType type, std::vector<Dim> dim_shape)
{
   AddIntermediateTensor(tensor_name, type, ConvertShapeToInt(dim_shape));
}

void RModel::AddOutputTensorNameList(std::vector<std::string> output_tensor_names)
{
   fOutputTensorNames.clear();
   for (auto &n : output_tensor_names) fOutputTensorNames.emplace_back(UTILITY::Clean_name(n));
}

void RModel::AddBlasRoutines(std::vector<std::string> routines)
{
   for (auto &r : routines) fNeededBlasRoutines.insert(r);
}

void RModel::AddNeededStdLib(std::string libname)
{
   if (fAllowedStdLib.count(libname)) fNeededStdLib.insert(libname);
}

// batchSize > 0 gives the parameters "input_size", "batch_size" and "bs" that value (RModel.cxx:398-407).
void RModel::Initialize(int batchSize, bool verbose)
{
   std::map<std::string, size_t> inputParams;
   if (batchSize > 0) {
      inputParams["input_size"] = batchSize;
      inputParams["batch_size"] = batchSize;
      inputParams["bs"] = batchSize;
   }
   Initialize(inputParams, verbose);
}

// Parametric input dimensions are replaced by the given values (a dimension named "<tensor>_size", which the
// parser makes out of a -1, answers to "input_size"), RModel.cxx:408-463. The reference goes on to emit
// shape-generic code for what is still parametric; the device emission sizes its buffers and launches at
// generation time, so a parameter without a value is an error here.
void RModel::Initialize(const std::map<std::string, size_t> &inputParams, bool verbose)
{
   fVerbose = int(verbose);
   if (fIsInitialized) return;
   auto parametric = fInputTensorInfos;
   for (auto &input : parametric) {
      const bool batchLed = !input.second.shape.empty() && input.second.shape[0].isParam;
      for (auto &d : input.second.shape) {
         if (!d.isParam) continue;
         std::string pname = d.param;
         if (pname == input.first + "_size") pname = "input_size";
         auto itr = inputParams.find(pname);
         if (itr != inputParams.end()) d = Dim{itr->second};
      }
      const std::vector<size_t> shape = ConvertShapeToInt(input.second.shape);
      if (shape.empty())
         throw std::runtime_error("TMVA-SOFIE: input tensor " + input.first + " has the parametric shape " +
                                  ConvertDynamicShapeToString(input.second.shape) +
                                  "; the device emission needs every dimension at generation time: pass the batch size "
                                  "to Generate / Initialize");
      fInputTensorInfos.erase(input.first);
      AddInputTensorInfo(input.first, input.second.type, shape);
      if (fRuntimeBatch && batchLed) {
         if (fBatchCapacity != 0 && fBatchCapacity != shape[0])
            throw std::runtime_error("TMVA-SOFIE: run-time batch: the inputs do not agree on the batch dimension");
         fBatchCapacity = shape[0];
         fBatchTensors.insert(UTILITY::Clean_name(input.first));
      }
   }
   if (fRuntimeBatch && fBatchTensors.empty())
      throw std::runtime_error("TMVA-SOFIE: Options::kRuntimeBatch needs an input whose leading dimension is a parameter");
   fIntermediateTensorInfos.clear();
   // every declared input must have a shape, as in the reference (RModel.cxx:410-468)
   for (auto &n : fInputTensorNames)
      if (!fReadyInputTensorInfos.count(n))
         throw std::runtime_error("TMVA-SOFIE: input tensor " + n + " has no shape information");
   if (fInputTensorNames.empty())
      for (auto &it : fReadyInputTensorInfos) fInputTensorNames.push_back(it.first);
   for (auto &op : fOperators) {
      op->Initialize(*this);
      if (!fRuntimeBatch) continue;
      // The batch travels along the first input of an operator: its outputs are then batch-led too and the
      // operator emits the Session's fBatch member where it would print the leading dimension.
      const auto &ins = op->GetOpInputTensors();
      for (size_t i = 1; i < ins.size(); ++i)
         if (fBatchTensors.count(ins[i]))
            throw std::runtime_error("TMVA-SOFIE: run-time batch: tensor " + ins[i] + " carries the batch but is not the first input of its " +
                                     op->Kind() + " operator");
      if (ins.empty() || !fBatchTensors.count(ins[0])) continue;
      if (!op->SetRuntimeBatch("fBatch", fBatchCapacity))
         throw std::runtime_error("TMVA-SOFIE: run-time batch: this " + op->Kind() + " operator cannot run on fewer rows than it is generated for");
      for (auto &out : op->GetOpOutputTensors()) {
         const auto shape = GetTensorShape(out);
         if (shape.empty() || shape[0] != fBatchCapacity)
            throw std::runtime_error("TMVA-SOFIE: run-time batch: tensor " + out + " loses the batch as its leading dimension");
         fBatchTensors.insert(out);
      }
   }
   for (auto &n : fOutputTensorNames)
      if (!CheckIfTensorAlreadyExist(n))
         throw std::runtime_error("TMVA-SOFIE: output tensor " + n + " is not produced by any operator");
   for (auto &n : fOutputTensorNames) {
      std::vector<size_t> chw;
      if (IsChannelsLast(n, &chw) && chw[0] > 1 && chw[1] * chw[2] > 1)
         throw std::runtime_error("TMVA-SOFIE: output tensor " + n + " is an int8 activation stored channels-last; "
                                  "end the graph with DequantizeLinear or a matrix product");
   }
   fIsInitialized = true;
}

// Float Conv followed by a BatchNormalization that is the only reader of its output: the normalisation is
// folded into the convolution's weights and bias at generation time and the BatchNormalization emits nothing.
// Runs before FuseActivations, so a Relu behind the pair is then fused into the convolution as usual.
void RModel::FuseBatchNorm()
{
   for (size_t i = 0; i + 1 < fOperators.size(); ++i) {
      auto *conv = dynamic_cast<ROperator_Conv<float> *>(fOperators[i].get());
      auto *bn = dynamic_cast<ROperator_BatchNormalization<float> *>(fOperators[i + 1].get());
      if (!conv || !bn || conv->GetOpOutputTensors().empty()) continue;
      const std::string mid = conv->GetOpOutputTensors()[0];
      if (bn->GetOpInputTensors().empty() || bn->GetOpInputTensors()[0] != mid) continue;
      bool other_use = std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), mid) != fOutputTensorNames.end();
      for (size_t j = 0; j < fOperators.size() && !other_use; ++j) {
         if (j == i + 1) continue;
         for (auto &in : fOperators[j]->GetOpInputTensors())
            if (in == mid) other_use = true;
      }
      if (other_use) continue;
      const std::string oldW = conv->WeightName(), oldB = conv->BiasName();
      if (!conv->FuseBatchNorm(*this, bn->FoldedScale(), bn->Mean(), bn->Bias(), bn->GetOpOutputTensors()[0], bn->HasActivation()))
         continue;
      bn->SetAbsorbed();
      fIntermediateTensorInfos.erase(mid);
      // initializers nobody reads any more are neither written to the weight file nor uploaded
      std::vector<std::string> orphans = bn->OwnInitializers();
      orphans.push_back(oldW);
      if (!oldB.empty()) orphans.push_back(oldB);
      for (auto &name : orphans) {
         bool used = false;
         for (size_t j = 0; j < fOperators.size() && !used; ++j) {
            if (j == i + 1) continue;
            for (auto &in : fOperators[j]->GetOpInputTensors())
               if (in == name) used = true;
         }
         if (!used && IsInitializedTensor(name)) SetNotWritableInitializedTensor(name);
      }
   }
}

// Conv / Gemm / QLinear* followed by a Relu that is the only consumer of their output:
// the activation moves into the producer's epilogue and the Relu becomes a view.
void RModel::FuseActivations()
{
   for (size_t j = 1; j < fOperators.size(); ++j) {
      ROperator &act = *fOperators[j];
      if (act.Kind() != "Relu" || act.GetOpInputTensors().empty()) continue;
      const std::string &mid = act.GetOpInputTensors()[0];
      // the operator that writes the activation's input (an absorbed operator writes nothing)
      size_t i = j;
      for (size_t k = 0; k < j; ++k) {
         if (fOperators[k]->IsAbsorbed() || fOperators[k]->GetOpOutputTensors().empty()) continue;
         if (fOperators[k]->GetOpOutputTensors()[0] == mid) i = k;
      }
      if (i == j) continue;
      bool other_use = std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), mid) != fOutputTensorNames.end();
      for (size_t k = 0; k < fOperators.size() && !other_use; ++k) {
         if (k == j || fOperators[k]->IsAbsorbed()) continue;
         for (auto &in : fOperators[k]->GetOpInputTensors())
            if (in == mid) other_use = true;
      }
      if (other_use) continue;
      if (fOperators[i]->FuseActivation(EActivationType::RELU)) act.SetFusedAway();
   }
}

// Gemm operators whose output feeds only the next Gemm (through a Relu that has moved into the producer's
// epilogue, if there is one) and whose matrices are small constants: a multilayer perceptron. The first operator of
// the chain emits one call for all layers (sofie_hip_mlp_f32), the others emit nothing, and the tensors between
// the layers stop existing. On a few hundred rows such a chain is bound by its launches, not by arithmetic.
void RModel::FuseGemmChain()
{
   auto readers_of = [&](const std::string &t) {
      std::vector<size_t> r;
      for (size_t k = 0; k < fOperators.size(); ++k) {
         if (fOperators[k]->IsAbsorbed()) continue;
         for (auto &in : fOperators[k]->GetOpInputTensors())
            if (in == t) { r.push_back(k); break; }
      }
      return r;
   };
   auto is_output = [&](const std::string &t) {
      return std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), t) != fOutputTensorNames.end();
   };
   for (size_t i = 0; i < fOperators.size(); ++i) {
      auto *head = dynamic_cast<ROperator_Gemm<float> *>(fOperators[i].get());
      if (!head || head->IsAbsorbed() || head->IsChainHead() || !head->ChainCandidate(*this)) continue;
      std::vector<ROperator_Gemm<float> *> layers = {head};
      std::vector<size_t> absorbed;            // operators that emit nothing any more
      std::vector<std::string> gone;           // tensors between the layers
      std::string cur = head->NameY();
      size_t work = head->MultiplyAdds();
      while (layers.size() < ROperator_Gemm<float>::kChainMaxLayers && !is_output(cur)) {
         const std::vector<size_t> readers = readers_of(cur);
         if (readers.size() != 1 || readers[0] <= i) break;
         ROperator &next = *fOperators[readers[0]];
         if (next.Kind() == "Relu" && next.IsFusedAway() && !next.GetOpOutputTensors().empty()) {
            // the activation already sits in the producer: its output is the same values under another name
            absorbed.push_back(readers[0]);
            gone.push_back(cur);
            cur = next.GetOpOutputTensors()[0];
            continue;
         }
         auto *g = dynamic_cast<ROperator_Gemm<float> *>(&next);
         if (!g || g->NameA() != cur || g->IsChainHead() || !g->ChainCandidate(*this)) break;
         // a transposed matrix is rewritten as [K, N]: only if this operator is its only reader
         if (g->TransB() && readers_of(g->NameB()).size() != 1) break;
         layers.push_back(g);
         absorbed.push_back(readers[0]);
         gone.push_back(cur);
         cur = g->NameY();
         work += g->MultiplyAdds();
      }
      // a trailing activation view that was walked over without a layer behind it stays what it was
      while (!absorbed.empty() && fOperators[absorbed.back()]->Kind() == "Relu") {
         cur = gone.back();
         absorbed.pop_back();
         gone.pop_back();
      }
      if (layers.size() < 2) continue;
      if (head->TransB() && readers_of(head->NameB()).size() != 1) continue;
      // past this much arithmetic the matrix-core kernels, one launch per layer, are the faster form
      if ((double)head->Rows() * (double)work > 536870912.0) continue;
      std::vector<ROperator_Gemm<float>::ChainLayer> chain;
      for (auto *g : layers) {
         g->MakeWeightsKByN(*this);
         chain.push_back(g->AsLayer());
      }
      head->BecomeChainHead(chain, cur);
      for (size_t k : absorbed) fOperators[k]->SetAbsorbed();
      for (auto &t : gone) fIntermediateTensorInfos.erase(t);
   }
}

// A QLinearMatMul whose int8 output feeds only a second, narrow QLinearMatMul (at most 8 columns: the last two
// layers of a classifier): the first operator emits one call for both (sofie_hip_qgemm_s8_pair), the second emits
// nothing. The tensor between them keeps its place in the pool: the library may use it, or skip it when it can
// apply the second layer in the pass that finishes the first.
void RModel::FuseQLinearPair()
{
   for (size_t i = 0; i < fOperators.size(); ++i) {
      auto *first = dynamic_cast<ROperator_QLinearMatMul *>(fOperators[i].get());
      if (!first || first->IsAbsorbed() || first->HasTail() || first->FloatOut()) continue;
      std::string cur = first->NameY();
      std::vector<size_t> views;
      ROperator_QLinearMatMul *second = nullptr;
      size_t at = 0;
      for (;;) {
         if (std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), cur) != fOutputTensorNames.end()) break;
         std::vector<size_t> readers;
         for (size_t k = 0; k < fOperators.size(); ++k) {
            if (fOperators[k]->IsAbsorbed()) continue;
            for (auto &in : fOperators[k]->GetOpInputTensors())
               if (in == cur) { readers.push_back(k); break; }
         }
         if (readers.size() != 1 || readers[0] <= i) break;
         ROperator &next = *fOperators[readers[0]];
         if (next.Kind() == "Relu" && next.IsFusedAway() && !next.GetOpOutputTensors().empty()) {
            views.push_back(readers[0]);
            cur = next.GetOpOutputTensors()[0];
            continue;
         }
         second = dynamic_cast<ROperator_QLinearMatMul *>(&next);
         at = readers[0];
         if (second && (second->NameA() != cur || second->HasTail() || second->Columns() > 8 || second->Depth() != first->Columns()))
            second = nullptr;
         break;
      }
      if (!second) continue;
      first->AppendTail(second->AsTail());
      second->SetAbsorbed();
      (void)at;
      (void)views;   // the activation views between the layers stay what they are: names for the first layer's tensor
   }
}

// Consecutive QLinearConv operators, each reading the (pooled) channels-last int8 output of the one before it, are
// emitted as one sofie_hip_qconv2d_s8_chain call by the first of them: the library then runs two layers in one launch
// where every workgroup owns the same images in both (no kernel boundary between them), and layer by layer otherwise,
// with the same bytes either way. Every layer's output stays a tensor of the model (the call writes them all), so
// other readers of them are served as before; the operators behind the first emit nothing.
void RModel::FuseQLinearConvChain()
{
   for (size_t i = 0; i < fOperators.size(); ++i) {
      auto *head = dynamic_cast<ROperator_QLinearConv *>(fOperators[i].get());
      if (!head || head->IsAbsorbed() || !head->ChainLayer()) continue;
      std::string cur = head->OutputName();
      for (size_t k = i + 1; k < fOperators.size() && head->ChainLength() < 8; ++k) {
         ROperator &op = *fOperators[k];
         if (op.IsAbsorbed() || op.IsFusedAway()) continue;      // emits nothing: a fused Relu, an absorbed MaxPool
         auto *next = dynamic_cast<ROperator_QLinearConv *>(&op);
         if (!next || !next->ChainLayer() || (next->InputName() != RootOf(cur) && next->InputName() != cur)) break;
         head->AppendLayer(*next);
         next->SetAbsorbed();
         cur = next->OutputName();
      }
   }
}

// QLinearConv (with its fused Relu) followed by a pad-free int8 MaxPool that is the only consumer of the
// activation: the pooling moves into the convolution call, which then writes the pooled tensor only.
// The unpooled tensors disappear from the model, the Relu and the MaxPool emit nothing.
void RModel::FusePooling()
{
   for (size_t i = 0; i + 1 < fOperators.size(); ++i) {
      ROperator &conv = *fOperators[i];
      if (conv.Kind() != "QLinearConv" || conv.GetOpOutputTensors().empty()) continue;
      std::vector<std::string> chain = {conv.GetOpOutputTensors()[0]};   // tensors that stop existing
      size_t j = i + 1;
      if (fOperators[j]->Kind() == "Relu" && fOperators[j]->IsFusedAway() && fOperators[j]->GetOpInputTensors()[0] == chain[0]) {
         chain.push_back(fOperators[j]->GetOpOutputTensors()[0]);
         ++j;
      }
      if (j >= fOperators.size() || fOperators[j]->Kind() != "Pool") continue;
      auto *pool = dynamic_cast<ROperator_Pool<float> *>(fOperators[j].get());
      if (!pool || !pool->IsPlainMaxPool() || pool->TensorType() != ETensorType::INT8) continue;
      if (pool->GetOpInputTensors()[0] != chain.back()) continue;
      // nobody else may read the unpooled tensors
      bool other_use = false;
      for (auto &t : chain) {
         if (std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), t) != fOutputTensorNames.end()) other_use = true;
         for (size_t k = 0; k < fOperators.size() && !other_use; ++k) {
            if (k == j || (k > i && k < j)) continue;
            for (auto &in : fOperators[k]->GetOpInputTensors())
               if (in == t) other_use = true;
         }
      }
      if (other_use) continue;
      if (!conv.FusePooling(pool->KernelShape(), pool->Strides(), pool->GetOpOutputTensors()[0], pool->OutputShape())) continue;
      for (size_t k = i + 1; k <= j; ++k) fOperators[k]->SetAbsorbed();
      for (auto &t : chain) {
         fIntermediateTensorInfos.erase(t);
         fChannelsLast.erase(t);
      }
   }
}

// QuantizeLinear whose int8 output is read by exactly one QLinearConv that can quantize its input itself
// (a first layer): the convolution reads the float tensor, the QuantizeLinear emits nothing and its output
// tensor disappears.
void RModel::FuseInputQuantization()
{
   for (size_t i = 0; i < fOperators.size(); ++i) {
      auto *q = dynamic_cast<ROperator_QuantizeLinear *>(fOperators[i].get());
      if (!q || q->IsAbsorbed() || q->GetOpOutputTensors().empty()) continue;
      const std::string &mid = q->GetOpOutputTensors()[0];
      if (std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), mid) != fOutputTensorNames.end()) continue;
      int consumer = -1, uses = 0;
      for (size_t j = 0; j < fOperators.size(); ++j) {
         if (j == i || fOperators[j]->IsAbsorbed()) continue;
         for (auto &in : fOperators[j]->GetOpInputTensors())
            if (in == mid) {
               ++uses;
               consumer = (int)j;
            }
      }
      if (uses != 1 || consumer < (int)i || fOperators[consumer]->Kind() != "QLinearConv") continue;
      if (!fOperators[consumer]->FuseInputQuantization(q->InputName(), q->Scale(), q->ZeroPoint())) continue;
      q->SetAbsorbed();
      fIntermediateTensorInfos.erase(mid);
      fChannelsLast.erase(mid);
   }
}

std::string RModel::RootOf(const std::string &name) const
{
   std::string r = name;
   for (auto it = fViewOf.find(r); it != fViewOf.end(); it = fViewOf.find(r)) r = it->second;
   return r;
}

// Lifetime of every intermediate = [index of its producer, index of its last consumer]; views
// extend the lifetime of the tensor they alias. Slots are assigned first-fit in producer order
// against all already-placed tensors whose lifetimes overlap (the reference's planner has the
// same goal, RModel.cxx:304-394, but tracks last use from incomplete operator input lists).
void RModel::PlanIntermediateMemory()
{
   fViewOf.clear();
   fPlacement.clear();
   for (auto &op : fOperators) {
      if (op->IsAbsorbed()) continue;
      std::string v = op->IsFusedAway() ? op->GetOpInputTensors()[0] : op->ViewOf();
      if (!v.empty() && !op->GetOpOutputTensors().empty() && fIntermediateTensorInfos.count(v))
         fViewOf[op->GetOpOutputTensors()[0]] = v;
   }
   const int nops = (int)fOperators.size();
   std::vector<std::string> order;
   for (int i = 0; i < nops; ++i) {
      for (auto &out : fOperators[i]->GetOpOutputTensors()) {
         if (!fIntermediateTensorInfos.count(out) || fViewOf.count(out) || fPlacement.count(out)) continue;
         Placement p;
         p.first = p.last = i;
         auto &info = fIntermediateTensorInfos[out];
         p.bytes = (ConvertShapeToLength(info.shape) * GetTypeSize(info.type) + 255) / 256 * 256;
         fPlacement[out] = p;
         order.push_back(out);
      }
   }
   for (int i = 0; i < nops; ++i)
      for (auto &in : fOperators[i]->GetOpInputTensors()) {
         auto f = fPlacement.find(RootOf(in));
         if (f != fPlacement.end() && i > f->second.last) f->second.last = i;
      }
   for (auto &n : fOutputTensorNames) {
      auto f = fPlacement.find(RootOf(n));
      if (f != fPlacement.end()) f->second.last = nops;
   }
   // intermediates registered by an operator but never listed as its output (none today) stay alive throughout
   for (auto &it : fIntermediateTensorInfos)
      if (!fPlacement.count(it.first) && !fViewOf.count(it.first)) {
         Placement p;
         p.first = 0;
         p.last = nops;
         p.bytes = (ConvertShapeToLength(it.second.shape) * GetTypeSize(it.second.type) + 255) / 256 * 256;
         fPlacement[it.first] = p;
         order.push_back(it.first);
      }
   fArenaBytes = 0;
   std::vector<std::string> placed;
   for (auto &name : order) {
      Placement &p = fPlacement[name];
      size_t off = 0;
      bool moved = true;
      while (moved) {
         moved = false;
         for (auto &other : placed) {
            const Placement &q = fPlacement[other];
            const bool time_overlap = p.first <= q.last && q.first <= p.last;
            const bool space_overlap = off < q.offset + q.bytes && q.offset < off + p.bytes;
            if (time_overlap && space_overlap) {
               off = q.offset + q.bytes;
               moved = true;
            }
         }
      }
      p.offset = off;
      placed.push_back(name);
      if (off + p.bytes > fArenaBytes) fArenaBytes = off + p.bytes;
   }
}

void RModel::GenerateHeaderInfo(std::string &hgname)
{
   fGC += "//Code generated automatically by SOFIE (MI355X device emission) from file " + fFileName +
          " at [" + fParseTime.substr(0, fParseTime.length() - 1) + "] \n";
   hgname = fName;
   std::transform(hgname.begin(), hgname.end(), hgname.begin(), [](unsigned char c) { return std::toupper(c); });
   hgname = "SOFIE_" + hgname;
   fGC += "\n#ifndef " + hgname + "\n";
   fGC += "#define " + hgname + "\n\n";
   for (auto &i : fNeededStdLib) fGC += "#include <" + i + ">\n";
   for (auto &i : fCustomOpHeaders) fGC += "#include \"" + i + "\"\n";
   fGC += "#include <cstdint>\n#include <cstring>\n#include <string>\n#include <stdexcept>\n#include <fstream>\n#include <tuple>\n#include <utility>\n";
   // the numerical library: a C ABI over device pointers instead of the reference's
   // extern "C" BLAS prototypes (RModel_Base.cxx:40-58)
   fGC += "#include \"sofie_hip.h\"\n";
   fGC += "\nnamespace SOFIE_" + fName + "{\n";
}

std::string RModel::GenerateInferSignature(bool isdecl)
{
   std::string rGC;
   int i_input = 0;
   for (auto &name : fInputTensorNames) {
      if (i_input++ > 0) rGC += ", ";
      if (isdecl) rGC += ConvertTypeToString(GetTensorType(name)) + "* ";
      rGC += "tensor_" + name;
   }
   return rGC;
}

void RModel::ReadInitializedTensorsFromFile(long /*pos*/)
{
   // Generated reader of the weight file. Text: "tensor_<name> <length>" then the values, with the
   // reference's name and length checks (RModel.cxx:970-1018); integer tensors use the same record layout
   // (the reference silently skips every non-float tensor, :1150-1152). Binary (the file starts with
   // "SOFIEBIN"): the same records as name, type and length fields followed by the raw little-endian values.
   // The format is recognised from the file, so a Session takes either.
   bool any = false;
   for (auto &i : fInitializedTensors) any |= i.second.IsWeightTensor();
   if (!any) return;
   fGC += "   std::ifstream f;\n";
   fGC += "   f.open(filename, std::ios::binary);\n";
   fGC += "   if (!f.is_open()) {\n";
   fGC += "      throw std::runtime_error(\"tmva-sofie failed to open file \" + filename + \" for input weights\");\n";
   fGC += "   }\n";
   fGC += "   const bool binary = IsBinaryWeightFile(f);\n";
   for (auto &i : fInitializedTensors) {
      if (!i.second.IsWeightTensor()) continue;
      const std::string tensor_name = "tensor_" + i.first;
      const std::string slength = std::to_string(ConvertShapeToLength(i.second.shape()));
      const std::string ctype = ConvertTypeToString(i.second.type());
      fGC += "   {\n";
      fGC += "      std::vector<" + ctype + "> host(" + slength + ");\n";
      fGC += "      ReadTensor(f, binary, \"" + tensor_name + "\", " + slength + ", " +
             std::to_string(static_cast<int>(i.second.type())) + ", host.data());\n";
      fGC += "      Check(sofie_hip_upload(fCtx, " + tensor_name + ", host.data(), " + slength + " * sizeof(" + ctype + ")), \"upload of " +
             tensor_name + "\");\n";
      fGC += "   }\n";
   }
   fGC += "   f.close();\n";
}

// Helpers of the generated Session that read one record of the weight file in either format.
std::string RModel::GenerateWeightReaderHelpers()
{
   std::string g;
   g += "static bool IsBinaryWeightFile(std::ifstream& f) {\n";
   g += "   char magic[8] = {0};\n";
   g += "   f.read(magic, 8);\n";
   g += "   if (f.gcount() == 8 && std::memcmp(magic, \"SOFIEBIN\", 8) == 0) {\n";
   g += "      uint32_t header[2] = {0, 0};   // format version, number of records\n";
   g += "      f.read(reinterpret_cast<char*>(header), sizeof(header));\n";
   g += "      if (f.fail() || header[0] != 1) throw std::runtime_error(\"TMVA-SOFIE binary weight file has an unknown version\");\n";
   g += "      return true;\n";
   g += "   }\n";
   g += "   f.clear();\n";
   g += "   f.seekg(0);\n";
   g += "   return false;\n";
   g += "}\n";
   g += "template <typename T>\n";
   g += "static void ReadTensor(std::ifstream& f, bool binary, const std::string& expected, size_t expected_length, unsigned expected_type, T* host) {\n";
   g += "   std::string tensor_name;\n";
   g += "   size_t length = 0;\n";
   g += "   if (binary) {\n";
   g += "      uint32_t name_length = 0, type = 0;\n";
   g += "      uint64_t count = 0;\n";
   g += "      f.read(reinterpret_cast<char*>(&name_length), 4);\n";
   g += "      if (f.fail() || name_length > 4096) throw std::runtime_error(\"TMVA-SOFIE failed to read the record of tensor \" + expected);\n";
   g += "      tensor_name.resize(name_length);\n";
   g += "      f.read(&tensor_name[0], name_length);\n";
   g += "      f.read(reinterpret_cast<char*>(&type), 4);\n";
   g += "      f.read(reinterpret_cast<char*>(&count), 8);\n";
   g += "      length = count;\n";
   g += "      // a record of the same name and count but another element type would be reinterpreted byte for byte\n";
   g += "      if (!f.fail() && tensor_name == expected && type != expected_type)\n";
   g += "         throw std::runtime_error(\"TMVA-SOFIE failed to read the correct tensor type for \" + expected + \"; expected type code is \" + std::to_string(expected_type) + \" , read \" + std::to_string(type));\n";
   g += "   } else {\n";
   g += "      f >> tensor_name >> length;\n";
   g += "   }\n";
   g += "   if (tensor_name != expected) {\n";
   g += "      std::string err_msg = \"TMVA-SOFIE failed to read the correct tensor name; expected name is \" + expected + \" , read \" + tensor_name;\n";
   g += "      throw std::runtime_error(err_msg);\n";
   g += "   }\n";
   g += "   if (length != expected_length) {\n";
   g += "      std::string err_msg = \"TMVA-SOFIE failed to read the correct tensor size; expected size is \" + std::to_string(expected_length) + \" , read \" + std::to_string(length);\n";
   g += "      throw std::runtime_error(err_msg);\n";
   g += "   }\n";
   g += "   if (binary) {\n";
   g += "      f.read(reinterpret_cast<char*>(host), length * sizeof(T));\n";
   g += "      const size_t pad = (8 - (length * sizeof(T)) % 8) % 8;   // records are padded to 8 bytes\n";
   g += "      f.ignore(pad);\n";
   g += "   } else if (sizeof(T) == 1) {\n";
   g += "      for (size_t i = 0; i < length; ++i) { int v; f >> v; host[i] = static_cast<T>(v); }   // bytes are written as numbers\n";
   g += "   } else {\n";
   g += "      for (size_t i = 0; i < length; ++i) f >> host[i];\n";
   g += "   }\n";
   g += "   if (f.fail()) {\n";
   g += "      throw std::runtime_error(\"TMVA-SOFIE failed to read the values for tensor \" + expected);\n";
   g += "   }\n";
   g += "}\n";
   return g;
}

// Binary weight file: "SOFIEBIN", u32 version (1), u32 record count, then per tensor u32 name length, the name
// ("tensor_<name>"), u32 element type (ETensorType), u64 element count, the raw values, zero padding to 8 bytes.
// Same order, names and subnormal flush as the text file.
long RModel::WriteInitializedTensorsToBinaryFile(std::string filename)
{
   if (filename == "") filename = fName + ".bin";
   std::ofstream f(filename, std::ios::binary);
   if (!f.is_open()) throw std::runtime_error("tmva-sofie failed to open file " + filename + " for tensor weight data");
   uint32_t count = 0;
   for (auto &i : fInitializedTensors) count += i.second.IsWeightTensor() ? 1 : 0;
   const uint32_t header[2] = {1, count};
   f.write("SOFIEBIN", 8);
   f.write(reinterpret_cast<const char *>(header), sizeof(header));
   for (auto &i : fInitializedTensors) {
      if (!i.second.IsWeightTensor()) continue;
      const std::string name = "tensor_" + i.first;
      const uint32_t name_length = (uint32_t)name.size(), type = (uint32_t)i.second.type();
      const uint64_t length = ConvertShapeToLength(i.second.shape());
      const size_t bytes = length * GetTypeSize(i.second.type());
      f.write(reinterpret_cast<const char *>(&name_length), 4);
      f.write(name.data(), name_length);
      f.write(reinterpret_cast<const char *>(&type), 4);
      f.write(reinterpret_cast<const char *>(&length), 8);
      if (i.second.type() == ETensorType::FLOAT) {
         std::vector<float> v(i.second.data<float>(), i.second.data<float>() + length);
         for (auto &x : v)
            if (x != 0. && std::abs(x) < std::numeric_limits<float>::min()) x = 0;
         f.write(reinterpret_cast<const char *>(v.data()), bytes);
      } else {
         f.write(reinterpret_cast<const char *>(i.second.data<char>()), bytes);
      }
      const char zeros[8] = {0};
      f.write(zeros, (8 - bytes % 8) % 8);
      if (f.fail()) throw std::runtime_error("tmva-sofie failed to write tensor data to file for " + name);
   }
   long pos = f.tellp();
   f.close();
   return pos;
}

long RModel::WriteInitializedTensorsToFile(std::string filename)
{
   if (filename == "") filename = fName + ".dat";
   std::ofstream f(filename);
   if (!f.is_open()) throw std::runtime_error("tmva-sofie failed to open file " + filename + " for tensor weight data");
   for (auto &i : fInitializedTensors) {
      if (!i.second.IsWeightTensor()) continue;
      const size_t length = ConvertShapeToLength(i.second.shape());
      f << "tensor_" << i.first << " " << length << "\n";
      for (size_t idx = 0; idx < length; idx++) {
         switch (i.second.type()) {
         case ETensorType::FLOAT: {
            // same text as the reference: max_digits10, subnormals flushed to zero (RModel.cxx:1140-1147)
            float value = i.second.data<float>()[idx];
            if (value != 0. && std::abs(value) < std::numeric_limits<float>::min()) value = 0;
            f << std::setprecision(std::numeric_limits<float>::max_digits10) << value;
            break;
         }
         case ETensorType::INT8: f << (int)i.second.data<int8_t>()[idx]; break;
         case ETensorType::UINT8:
         case ETensorType::FLOAT8E4M3FN: f << (int)i.second.data<uint8_t>()[idx]; break;
         case ETensorType::INT32: f << i.second.data<int32_t>()[idx]; break;
         case ETensorType::INT64: f << i.second.data<int64_t>()[idx]; break;
         default:
            throw std::runtime_error("tmva-sofie tensor tensor_" + i.first + " with type " +
                                     ConvertTypeToString(i.second.type()) + " cannot be written to a file");
         }
         f << ((idx < length - 1) ? " " : "\n");
      }
      if (length == 0) f << "\n";
      if (f.fail()) throw std::runtime_error("tmva-sofie failed to write tensor data to file for tensor_" + i.first);
   }
   long pos = f.tellp();
   f.close();
   return pos;
}

void RModel::GenerateSessionCode()
{
   fGC += "struct Session {\n";
   fGC += "// the context handle empties its source when moved, so a moved-from Session releases nothing\n";
   fGC += "struct CtxHandle {\n";
   fGC += "   sofie_hip_ctx* p = nullptr;\n";
   fGC += "   CtxHandle() = default;\n";
   fGC += "   CtxHandle(CtxHandle&& o) noexcept : p(o.p) { o.p = nullptr; }\n";
   fGC += "   CtxHandle& operator=(CtxHandle&&) = delete;\n";
   fGC += "   operator sofie_hip_ctx*() const { return p; }\n";
   fGC += "};\n";
   fGC += "CtxHandle fCtx;\n";
   fGC += "sofie_hip_graph* fGraph = nullptr;   // the operator sequence on the Session's own input buffer, recorded once\n";
   fGC += "bool fUseGraph = false;\n";
   if (fRuntimeBatch)
      fGC += "size_t fBatch = " + std::to_string(fBatchCapacity) + ";   // rows of the batch the operators process, at most " +
             std::to_string(fBatchCapacity) + " (the capacity every buffer is sized for)\n";
   fGC += "static void Check(sofie_hip_ctx* ctx, int status, const char* what) {\n";
   fGC += "   if (status != 0) throw std::runtime_error(std::string(\"TMVA SOFIE device error in \") + what + \": \" + "
          "sofie_hip_last_error(ctx));\n";
   fGC += "}\n";
   fGC += "void Check(int status, const char* what) { Check(fCtx, status, what); }\n";
   {
      bool any = false;
      for (auto &i : fInitializedTensors) any |= i.second.IsWeightTensor();
      if (any && fUseWeightFile) fGC += GenerateWeightReaderHelpers();
   }
   // weights: device pointers, uploaded once in the constructor
   for (auto &i : fInitializedTensors) {
      if (!i.second.IsWeightTensor()) continue;   // folded into other tensors at generation time
      const std::string ctype = ConvertTypeToString(i.second.type());
      fGC += ctype + " * tensor_" + i.first + " = nullptr;   // device, " +
             std::to_string(ConvertShapeToLength(i.second.shape())) + " elements\n";
   }
   // inputs: device staging buffers for the host-pointer infer()
   for (auto &n : fInputTensorNames) {
      fGC += ConvertTypeToString(GetTensorType(n)) + " * fInput_" + n + " = nullptr;   // device copy of the input\n";
      fGC += ConvertTypeToString(GetTensorType(n)) + " * fPinned_" + n + " = nullptr;   // page-locked host buffer, made on request\n";
   }
   // intermediates: one device arena, offsets from the memory plan
   fGC += "char* fIntermediateMemoryPool = nullptr;   // device, " + std::to_string(fArenaBytes) + " bytes\n";
   for (auto &it : fIntermediateTensorInfos)
      fGC += ConvertTypeToString(it.second.type) + " * tensor_" + it.first + " = nullptr;\n";
   for (size_t id = 0; id < fOperators.size(); id++) fGC += fOperators[id]->GenerateSessionMembersCode(std::to_string(id));
   fGC += "\n";

   // ---- constructor
   fGC += "Session(std::string filename =\"" +
          (fUseWeightFile ? fName + (fWeightFile == WeightFileType::Binary ? ".bin" : ".dat") : std::string("")) +
          "\", int device = 0) {\n";
   {
      bool reads_file = false;
      for (auto &i : fInitializedTensors) reads_file = reads_file || (fUseWeightFile && i.second.IsWeightTensor());
      if (!reads_file) fGC += "   (void)filename;   // no weight file is read\n";
   }
   fGC += "   { int status = sofie_hip_create(&fCtx.p, device, nullptr);\n";
   fGC += "     if (status != 0) throw std::runtime_error(\"TMVA SOFIE cannot create a device context\"); }\n";
   fGC += "   try {\n";
   // the weights are uploaded below and never written again: the library may keep its own layouts of them
   fGC += "   Check(sofie_hip_constant_weights(fCtx, 1), \"Session construction\");\n";
   for (auto &i : fInitializedTensors) {
      if (!i.second.IsWeightTensor()) continue;
      const size_t bytes = ConvertShapeToLength(i.second.shape()) * GetTypeSize(i.second.type());
      fGC += "   Check(sofie_hip_malloc(fCtx, reinterpret_cast<void**>(&tensor_" + i.first + "), " + std::to_string(bytes) +
             "), \"allocation of tensor_" + i.first + "\");\n";
   }
   for (auto &n : fInputTensorNames) {
      const size_t bytes = ConvertShapeToLength(GetTensorShape(n)) * GetTypeSize(GetTensorType(n));
      fGC += "   Check(sofie_hip_malloc(fCtx, reinterpret_cast<void**>(&fInput_" + n + "), " + std::to_string(bytes) +
             "), \"allocation of the input buffer\");\n";
   }
   fGC += "   Check(sofie_hip_malloc(fCtx, reinterpret_cast<void**>(&fIntermediateMemoryPool), " +
          std::to_string(fArenaBytes) + "), \"allocation of the intermediate pool\");\n";
   for (auto &it : fIntermediateTensorInfos) {
      if (fViewOf.count(it.first)) continue;
      fGC += "   tensor_" + it.first + " = reinterpret_cast<" + ConvertTypeToString(it.second.type) +
             "*>(fIntermediateMemoryPool + " + std::to_string(fPlacement[it.first].offset) + ");\n";
   }
   // views after their roots
   for (auto &op : fOperators)
      for (auto &out : op->GetOpOutputTensors()) {
         auto v = fViewOf.find(out);
         if (v == fViewOf.end()) continue;
         fGC += "   tensor_" + out + " = reinterpret_cast<" + ConvertTypeToString(fIntermediateTensorInfos[out].type) +
                "*>(tensor_" + v->second + ");\n";
      }
   if (fUseWeightFile) {
      ReadInitializedTensorsFromFile(0);
   } else {
      for (auto &i : fInitializedTensors) {
         if (!i.second.IsWeightTensor()) continue;
         const std::string ctype = ConvertTypeToString(i.second.type());
         const size_t length = ConvertShapeToLength(i.second.shape());
         std::stringstream lit;
         lit << "   { static const " << ctype << " host[" << (length ? length : 1) << "] = {";
         for (size_t idx = 0; idx < length; ++idx) {
            if (idx) lit << ", ";
            switch (i.second.type()) {
            case ETensorType::FLOAT:
            {
               std::stringstream one;
               one << std::setprecision(std::numeric_limits<float>::max_digits10) << i.second.data<float>()[idx];
               std::string text = one.str();
               if (!std::isfinite(i.second.data<float>()[idx]))
                  throw std::runtime_error("tmva-sofie tensor_" + i.first + " holds a non-finite value");
               // a float literal needs a '.' or an exponent before its suffix
               if (text.find_first_of(".e") == std::string::npos) text += ".";
               lit << text << "f";
               break;
            }
            case ETensorType::INT8: lit << (int)i.second.data<int8_t>()[idx]; break;
            case ETensorType::UINT8:
            case ETensorType::FLOAT8E4M3FN: lit << (int)i.second.data<uint8_t>()[idx]; break;
            case ETensorType::INT32: lit << i.second.data<int32_t>()[idx]; break;
            case ETensorType::INT64: lit << i.second.data<int64_t>()[idx]; break;
            default: throw std::runtime_error("tmva-sofie tensor_" + i.first + " cannot be written as a literal");
            }
         }
         lit << "};\n     Check(sofie_hip_upload(fCtx, tensor_" << i.first << ", host, " << length * GetTypeSize(i.second.type())
             << "), \"upload of tensor_" << i.first << "\"); }\n";
         fGC += lit.str();
      }
   }
   for (size_t id = 0; id < fOperators.size(); id++) fGC += fOperators[id]->GenerateInitCode();
   fGC += "   Check(sofie_hip_sync(fCtx), \"Session construction\");\n";
   fGC += "   } catch (...) { Release(); throw; }\n";
   fGC += "}\n\n";

   // ---- destructor (the reference's Session leaks its pool; device memory must not)
   fGC += "void Release() {\n";
   fGC += "   if (!fCtx) return;\n";
   fGC += "   sofie_hip_graph_destroy(fCtx, fGraph);\n";
   fGC += "   fGraph = nullptr;\n";
   for (auto &i : fInitializedTensors)
      if (i.second.IsWeightTensor()) fGC += "   sofie_hip_free(fCtx, tensor_" + i.first + ");\n";
   for (auto &n : fInputTensorNames) fGC += "   sofie_hip_free(fCtx, fInput_" + n + ");\n";
   for (auto &n : fInputTensorNames) fGC += "   sofie_hip_host_free(fCtx, fPinned_" + n + ");\n";
   fGC += "   sofie_hip_free(fCtx, fIntermediateMemoryPool);\n";
   fGC += "   sofie_hip_destroy(fCtx);\n";
   fGC += "   fCtx.p = nullptr;\n";
   fGC += "}\n";
   // page-locked host buffers of the inputs' size: a caller that fills them and passes the same pointer to infer()
   // gets the upload at the rate of the link (pageable memory goes through the driver's staging copy first)
   for (auto &n : fInputTensorNames) {
      const std::string t = ConvertTypeToString(GetTensorType(n));
      const size_t bytes = ConvertShapeToLength(GetTensorShape(n)) * GetTypeSize(GetTensorType(n));
      fGC += t + "* pinned_input_" + n + "() {\n";
      fGC += "   if (!fPinned_" + n + ") Check(sofie_hip_host_malloc(fCtx, reinterpret_cast<void**>(&fPinned_" + n + "), " +
             std::to_string(bytes) + "), \"allocation of a page-locked input buffer\");\n";
      fGC += "   return fPinned_" + n + ";\n";
      fGC += "}\n";
   }
   fGC += "~Session() { Release(); }\n";
   fGC += "Session(const Session&) = delete;\n";
   fGC += "Session& operator=(const Session&) = delete;\n";
   fGC += "Session(Session&&) noexcept = default;   // containers of Sessions (SofieFunctor) need it\n\n";

   // ---- the operator sequence on device pointers
   fGC += "// every argument is a device pointer; kernels are enqueued on the Session's stream\n";
   fGC += "void run_device(";
   {
      int k = 0;
      for (auto &n : fInputTensorNames) {
         if (k++) fGC += ", ";
         fGC += "const " + ConvertTypeToString(GetTensorType(n)) + "* tensor_" + n;
      }
   }
   fGC += "){\n";
   for (size_t id = 0; id < fOperators.size(); id++) {
      if (fOperators[id]->IsFusedAway() || fOperators[id]->IsAbsorbed()) continue;
      fGC += fOperators[id]->Generate(std::to_string(id));
   }
   fGC += "}\n\n";

   // ---- return convention of infer(), as in the reference (RModel.cxx:744-801): one output is a std::vector of its
   // type; several outputs of one type are a std::vector of std::vectors; outputs of different types are a
   // std::tuple of std::vectors, all in the order of the output list
   const size_t nout = fOutputTensorNames.size();
   if (nout == 0) throw std::runtime_error("TMVA-SOFIE: output size=0 are not supported");
   const std::string out = fOutputTensorNames[0];
   const std::string otype = ConvertTypeToString(GetTensorType(out));
   bool sameOutputTypes = true;
   for (auto &n : fOutputTensorNames) sameOutputTypes = sameOutputTypes && GetTensorType(n) == GetTensorType(out);
   std::string inferReturnType = "std::vector<" + otype + ">";
   std::string deviceReturnType = "const " + otype + "*";
   if (nout > 1) {
      if (sameOutputTypes) {
         inferReturnType = "std::vector<std::vector<" + otype + ">>";
      } else {
         inferReturnType = "std::tuple<";
         for (size_t i = 0; i < nout; ++i)
            inferReturnType += std::string(i ? "," : "") + "std::vector<" + ConvertTypeToString(GetTensorType(fOutputTensorNames[i])) + ">";
         inferReturnType += ">";
      }
      deviceReturnType = "std::tuple<";
      for (size_t i = 0; i < nout; ++i)
         deviceReturnType += std::string(i ? "," : "") + "const " + ConvertTypeToString(GetTensorType(fOutputTensorNames[i])) + "*";
      deviceReturnType += ">";
   }
   // element count of output i as the generated code states it (rows of the current batch with a run-time batch)
   auto outputCount = [&](const std::string &n) {
      const size_t len = ConvertShapeToLength(GetTensorShape(n));
      return (fRuntimeBatch && fBatchTensors.count(n)) ? "fBatch * " + std::to_string(len / fBatchCapacity) : std::to_string(len);
   };
   // the statements that download every output and return them
   auto downloads = [&]() {
      if (nout == 1) {
         fGC += "   std::vector<" + otype + "> ret(" + outputCount(out) + ");\n";
         fGC += "   Check(sofie_hip_download(fCtx, ret.data(), tensor_" + out + ", ret.size() * sizeof(" + otype + ")), \"output download\");\n";
         fGC += "   return ret;\n";
         return;
      }
      for (size_t i = 0; i < nout; ++i) {
         const std::string &n = fOutputTensorNames[i];
         const std::string t = ConvertTypeToString(GetTensorType(n));
         const std::string v = "ret_" + std::to_string(i);
         fGC += "   std::vector<" + t + "> " + v + "(" + outputCount(n) + ");\n";
         fGC += "   Check(sofie_hip_download(fCtx, " + v + ".data(), tensor_" + n + ", " + v + ".size() * sizeof(" + t + ")), \"output download\");\n";
      }
      fGC += "   return " + inferReturnType + "{";
      for (size_t i = 0; i < nout; ++i) fGC += std::string(i ? ", " : "") + "std::move(ret_" + std::to_string(i) + ")";
      fGC += "};\n";
   };

   // ---- the sequence on the Session's own input buffer, optionally replayed from a HIP graph
   {
      std::string own;
      int k = 0;
      for (auto &n : fInputTensorNames) own += std::string(k++ ? ", " : "") + "fInput_" + n;
      fGC += "// use_graph(true): infer() replays the operator sequence from a HIP graph recorded at the first call (one\n";
      fGC += "// submission instead of one per operator; worth it for chains of small kernels). The first call runs the\n";
      fGC += "// sequence once eagerly, so that nothing allocates while it is recorded.\n";
      fGC += "void use_graph(bool on = true) { fUseGraph = on; }\n";
      fGC += "void run_own_input() {\n";
      fGC += "   if (!fUseGraph) { run_device(" + own + "); return; }\n";
      fGC += "   if (!fGraph) {\n";
      fGC += "      run_device(" + own + ");\n";
      fGC += "      Check(sofie_hip_capture_begin(fCtx), \"graph capture\");\n";
      fGC += "      try { run_device(" + own + "); } catch (...) { sofie_hip_capture_end(fCtx, nullptr); throw; }\n";
      fGC += "      Check(sofie_hip_capture_end(fCtx, &fGraph), \"graph capture\");\n";
      fGC += "   }\n";
      fGC += "   Check(sofie_hip_graph_launch(fCtx, fGraph), \"graph launch\");\n";
      fGC += "}\n\n";
   }

   // ---- infer on host pointers: same signature and return convention as the reference
   // (RModel.cxx:680-801): one upload, the kernel sequence, one download
   auto uploads = [&]() {
      for (auto &n : fInputTensorNames) {
         const size_t bytes = ConvertShapeToLength(GetTensorShape(n)) * GetTypeSize(GetTensorType(n));
         const std::string count = (fRuntimeBatch && fBatchTensors.count(n)) ? "fBatch * " + std::to_string(bytes / fBatchCapacity)
                                                                            : std::to_string(bytes);
         fGC += "   Check(sofie_hip_upload(fCtx, fInput_" + n + ", tensor_" + n + ", " + count + "), \"input upload\");\n";
      }
   };
   if (fRuntimeBatch) {
      fGC += "// the batch the next run processes: any value from 1 to the capacity of " + std::to_string(fBatchCapacity) + "\n";
      fGC += "void set_batch(size_t batch) {\n";
      fGC += "   if (batch == 0 || batch > " + std::to_string(fBatchCapacity) +
             ") throw std::runtime_error(\"TMVA SOFIE: the batch must be between 1 and " + std::to_string(fBatchCapacity) +
             ", the size this Session was generated for\");\n";
      fGC += "   if (batch != fBatch && fGraph) { sofie_hip_graph_destroy(fCtx, fGraph); fGraph = nullptr; }   // recorded for another size\n";
      fGC += "   fBatch = batch;\n";
      fGC += "}\n";
      fGC += "// infer on the first `batch` rows of the inputs; returns that many rows\n";
      fGC += inferReturnType + " infer(size_t batch, " + GenerateInferSignature(true) + "){\n";
      fGC += "   set_batch(batch);\n";
      uploads();
      fGC += "   run_own_input();\n";
      downloads();
      fGC += "}\n";
      fGC += "// the whole capacity, as a Session generated for a fixed batch\n";
      fGC += inferReturnType + " infer(" + GenerateInferSignature(true) + "){ return infer(" + std::to_string(fBatchCapacity) +
             ", " + GenerateInferSignature(false) + "); }\n\n";
   } else {
      fGC += inferReturnType + " infer(" + GenerateInferSignature(true) + "){\n";
      uploads();
      fGC += "   run_own_input();\n";
      downloads();
      fGC += "}\n\n";
   }

   // ---- infer on device pointers: nothing crosses PCIe; returns the device address of the output (a tuple of the
   // addresses, in the order of the output list, when there are several)
   fGC += deviceReturnType + " infer_device(";
   {
      int k = 0;
      for (auto &n : fInputTensorNames) {
         if (k++) fGC += ", ";
         fGC += "const " + ConvertTypeToString(GetTensorType(n)) + "* tensor_" + n;
      }
   }
   fGC += "){\n   run_device(";
   {
      int k = 0;
      for (auto &n : fInputTensorNames) fGC += std::string(k++ ? ", " : "") + "tensor_" + n;
   }
   fGC += ");\n   return ";
   if (nout == 1) {
      fGC += "tensor_" + out;
   } else {
      fGC += deviceReturnType + "{";
      for (size_t i = 0; i < nout; ++i) fGC += std::string(i ? ", " : "") + "tensor_" + fOutputTensorNames[i];
      fGC += "}";
   }
   fGC += ";\n}\n";
   fGC += "void sync() { Check(sofie_hip_sync(fCtx), \"sync\"); }\n";
   fGC += "};\n";
}

// ---- Options::kHostCode: the Session for the host cores, as the reference generates it (RModel.cxx:560-801 there):
// weights and intermediates in host memory, operators as BLAS calls and loops, infer(float*...) returning vectors.
void RModel::GenerateHostHeaderInfo(std::string &hgname)
{
   fGC += "//Code generated automatically by SOFIE (host emission) from file " + fFileName + " at [" +
          fParseTime.substr(0, fParseTime.length() - 1) + "] \n";
   hgname = fName;
   std::transform(hgname.begin(), hgname.end(), hgname.begin(), [](unsigned char c) { return std::toupper(c); });
   hgname = "SOFIE_" + hgname;
   fGC += "\n#ifndef " + hgname + "\n";
   fGC += "#define " + hgname + "\n\n";
   for (auto &i : fNeededStdLib) fGC += "#include <" + i + ">\n";
   fGC += "#include <algorithm>\n#include <cmath>\n#include <cstdint>\n#include <cstring>\n#include <string>\n#include <stdexcept>\n#include <fstream>\n"
          "#include <tuple>\n#include <utility>\n#include <limits>\n";
   fGC += "\nnamespace SOFIE_" + fName + "{\n";
   // the Fortran BLAS the program is linked with, declared as the reference declares it (RModel_Base.cxx:40-58)
   fGC += "namespace BLAS{\n";
   fGC += "   extern \"C\" void sgemm_(const char * transa, const char * transb, const int * m, const int * n, const int * k,\n"
          "                          const float * alpha, const float * A, const int * lda, const float * B, const int * ldb,\n"
          "                          const float * beta, float * C, const int * ldc);\n";
   fGC += "   extern \"C\" void saxpy_(const int * n, const float * alpha, const float * x, const int * incx, float * y, const int * incy);\n";
   fGC += "}//BLAS\n";
   // Patches of one image (or one group's channels of it) as a column-major [output positions, C * kernel cells]
   // matrix over three spatial axes (extent 1 for missing leading ones): a column holds, for every output position,
   // the input cell under one kernel cell of one channel, zero outside the image (the role of UTILITY::Im2col and
   // Im2col_3d of the reference, SOFIE_common.hxx:485-518).
   fGC += "inline void Im2col(const float * x, int C, const int * in, const int * kernel, const int * pads, const int * strides,\n"
          "                   const int * dilations, const int * out, float * xcol) {\n"
          "   const size_t outSize = static_cast<size_t>(out[0]) * out[1] * out[2];\n"
          "   size_t column = 0;\n"
          "   for (int c = 0; c < C; ++c)\n"
          "      for (int kd = 0; kd < kernel[0]; ++kd)\n"
          "         for (int kh = 0; kh < kernel[1]; ++kh)\n"
          "            for (int kw = 0; kw < kernel[2]; ++kw, ++column) {\n"
          "               float * col = xcol + column * outSize;\n"
          "               for (int od = 0; od < out[0]; ++od) {\n"
          "                  const int id = od * strides[0] - pads[0] + kd * dilations[0];\n"
          "                  for (int oh = 0; oh < out[1]; ++oh) {\n"
          "                     const int ih = oh * strides[1] - pads[1] + kh * dilations[1];\n"
          "                     if (id < 0 || id >= in[0] || ih < 0 || ih >= in[1]) {\n"
          "                        for (int ow = 0; ow < out[2]; ++ow) *col++ = 0.f;\n"
          "                        continue;\n"
          "                     }\n"
          "                     const float * row = x + ((static_cast<size_t>(c) * in[0] + id) * in[1] + ih) * in[2];\n"
          "                     int iw = kw * dilations[2] - pads[2];\n"
          "                     for (int ow = 0; ow < out[2]; ++ow, iw += strides[2]) *col++ = (iw >= 0 && iw < in[2]) ? row[iw] : 0.f;\n"
          "                  }\n"
          "               }\n"
          "            }\n"
          "}\n";
   // The other way round, for the transposed convolution: column (oc*KH + kh)*KW + kw of a column-major
   // [H*W, OC*KH*KW] matrix is added into channel oc of the output at the positions kernel cell (kh, kw) reaches.
   fGC += "inline void Col2im(const float * col, int OC, int H, int W, int KH, int KW, int padTop, int padLeft, int strideH, int strideW,\n"
          "                   int dilationH, int dilationW, int OH, int OW, float * y) {\n"
          "   for (int oc = 0; oc < OC; ++oc)\n"
          "      for (int kh = 0; kh < KH; ++kh)\n"
          "         for (int kw = 0; kw < KW; ++kw) {\n"
          "            const float * c = col + (static_cast<size_t>(oc * KH + kh) * KW + kw) * H * W;\n"
          "            for (int ih = 0; ih < H; ++ih) {\n"
          "               const int oh = ih * strideH - padTop + kh * dilationH;\n"
          "               if (oh < 0 || oh >= OH) continue;\n"
          "               for (int iw = 0; iw < W; ++iw) {\n"
          "                  const int ow = iw * strideW - padLeft + kw * dilationW;\n"
          "                  if (ow >= 0 && ow < OW) y[(static_cast<size_t>(oc) * OH + oh) * OW + ow] += c[ih * W + iw];\n"
          "               }\n"
          "            }\n"
          "         }\n"
          "}\n";
   // Einsum as loops: labels 0 .. nOut-1 index the output (row-major), the others are summed, innermost last;
   // stride[i*nLabels + l] is operand i's element stride along label l (0 where the operand lacks it).
   fGC += "inline void EinsumLoops(int nInputs, const float * const * x, int nLabels, int nOut, const int * extent, const long long * stride,\n"
          "                        float * y) {\n"
          "   std::vector<int> pos(nLabels > 0 ? nLabels : 1, 0);\n"
          "   size_t outputs = 1, terms = 1;\n"
          "   for (int l = 0; l < nOut; ++l) outputs *= extent[l];\n"
          "   for (int l = nOut; l < nLabels; ++l) terms *= extent[l];\n"
          "   for (size_t o = 0; o < outputs; ++o) {\n"
          "      float sum = 0.f;\n"
          "      for (int l = nOut; l < nLabels; ++l) pos[l] = 0;\n"
          "      for (size_t t = 0; t < terms; ++t) {\n"
          "         float product = 1.f;\n"
          "         for (int i = 0; i < nInputs; ++i) {\n"
          "            long long at = 0;\n"
          "            for (int l = 0; l < nLabels; ++l) at += pos[l] * stride[i * nLabels + l];\n"
          "            product *= x[i][at];\n"
          "         }\n"
          "         sum += product;\n"
          "         for (int l = nLabels - 1; l >= nOut; --l) { if (++pos[l] < extent[l]) break; pos[l] = 0; }\n"
          "      }\n"
          "      y[o] = sum;\n"
          "      for (int l = nOut - 1; l >= 0; --l) { if (++pos[l] < extent[l]) break; pos[l] = 0; }\n"
          "   }\n"
          "}\n";
   // The quantized operators' arithmetic, one value at a time: round half to even in fp32 (the default rounding mode),
   // the rounded value kept inside +-1024 so that the conversion to int is defined, saturation to int8; a ReLU behind a
   // quantized operator is a lower clamp at the output zero-point.
   fGC += "inline int8_t Requantize(int32_t acc, float scale, int zeroPoint, bool relu) {\n"
          "   float r = std::nearbyint(static_cast<float>(acc) * scale);\n"
          "   r = r > 1024.f ? 1024.f : (r < -1024.f ? -1024.f : r);\n"
          "   int q = static_cast<int>(r) + zeroPoint;\n"
          "   const int lo = (relu && zeroPoint > -128) ? zeroPoint : -128;\n"
          "   q = q < lo ? lo : (q > 127 ? 127 : q);\n"
          "   return static_cast<int8_t>(q);\n"
          "}\n";
   fGC += "inline int8_t QuantizeOne(float x, float scale, int zeroPoint) {\n"
          "   float r = std::nearbyint(x / scale);\n"
          "   r = r > 1024.f ? 1024.f : (r < -1024.f ? -1024.f : r);\n"
          "   int q = static_cast<int>(r) + zeroPoint;\n"
          "   q = q < -128 ? -128 : (q > 127 ? 127 : q);\n"
          "   return static_cast<int8_t>(q);\n"
          "}\n";
   fGC += "inline void MaxPoolInt8(const int8_t * x, int8_t * y, size_t N, size_t C, size_t H, size_t W, size_t KH, size_t KW, size_t padTop,\n"
          "                        size_t padLeft, size_t strideH, size_t strideW, size_t OH, size_t OW, bool channelsLast) {\n"
          "   for (size_t n = 0; n < N; ++n)\n"
          "      for (size_t c = 0; c < C; ++c)\n"
          "         for (size_t oh = 0; oh < OH; ++oh)\n"
          "            for (size_t ow = 0; ow < OW; ++ow) {\n"
          "               int best = -128;\n"
          "               for (size_t kh = 0; kh < KH; ++kh) {\n"
          "                  const long ih = static_cast<long>(oh * strideH + kh) - static_cast<long>(padTop);\n"
          "                  if (ih < 0 || ih >= static_cast<long>(H)) continue;\n"
          "                  for (size_t kw = 0; kw < KW; ++kw) {\n"
          "                     const long iw = static_cast<long>(ow * strideW + kw) - static_cast<long>(padLeft);\n"
          "                     if (iw < 0 || iw >= static_cast<long>(W)) continue;\n"
          "                     const int v = channelsLast ? x[((n * H + ih) * W + iw) * C + c] : x[((n * C + c) * H + ih) * W + iw];\n"
          "                     if (v > best) best = v;\n"
          "                  }\n"
          "               }\n"
          "               y[channelsLast ? ((n * OH + oh) * OW + ow) * C + c : ((n * C + c) * OH + oh) * OW + ow] = static_cast<int8_t>(best);\n"
          "            }\n"
          "}\n";
   // Pooling over three axes (leading axes of extent 1 for fewer): maximum, or mean, of the window's cells inside the image.
   fGC += "inline void Pool3d(bool isMax, bool countIncludePad, const float * x, float * y, size_t planes, const int * in, const int * out,\n"
          "                   const int * kernel, const int * pads, const int * strides) {\n"
          "   const size_t inSize = static_cast<size_t>(in[0]) * in[1] * in[2];\n"
          "   size_t o = 0;\n"
          "   for (size_t p = 0; p < planes; ++p) {\n"
          "      const float * xp = x + p * inSize;\n"
          "      for (int od = 0; od < out[0]; ++od)\n"
          "         for (int oh = 0; oh < out[1]; ++oh)\n"
          "            for (int ow = 0; ow < out[2]; ++ow) {\n"
          "               float value = isMax ? -std::numeric_limits<float>::infinity() : 0.f;\n"
          "               int cells = 0;\n"
          "               for (int kd = 0; kd < kernel[0]; ++kd) {\n"
          "                  const int id = od * strides[0] - pads[0] + kd;\n"
          "                  if (id < 0 || id >= in[0]) continue;\n"
          "                  for (int kh = 0; kh < kernel[1]; ++kh) {\n"
          "                     const int ih = oh * strides[1] - pads[1] + kh;\n"
          "                     if (ih < 0 || ih >= in[1]) continue;\n"
          "                     for (int kw = 0; kw < kernel[2]; ++kw) {\n"
          "                        const int iw = ow * strides[2] - pads[2] + kw;\n"
          "                        if (iw < 0 || iw >= in[2]) continue;\n"
          "                        const float v = xp[(static_cast<size_t>(id) * in[1] + ih) * in[2] + iw];\n"
          "                        if (isMax) { if (v > value) value = v; } else value += v;\n"
          "                        cells++;\n"
          "                     }\n"
          "                  }\n"
          "               }\n"
          "               if (!isMax) value /= static_cast<float>(countIncludePad ? kernel[0] * kernel[1] * kernel[2] : cells);\n"
          "               y[o++] = value;\n"
          "            }\n"
          "   }\n"
          "}\n";
}

void RModel::GenerateHostSessionCode()
{
   fGC += "struct Session {\n";
   if (fRuntimeBatch)
      fGC += "size_t fBatch = " + std::to_string(fBatchCapacity) + ";   // rows of the batch the operators process, at most " +
             std::to_string(fBatchCapacity) + "\n";
   {
      bool any = false;
      for (auto &i : fInitializedTensors) any |= i.second.IsWeightTensor();
      if (any && fUseWeightFile) fGC += GenerateWeightReaderHelpers();
   }
   for (auto &i : fInitializedTensors) {
      if (!i.second.IsWeightTensor()) continue;
      const std::string ctype = ConvertTypeToString(i.second.type());
      const size_t length = ConvertShapeToLength(i.second.shape());
      fGC += "std::vector<" + ctype + "> fTensor_" + i.first + " = std::vector<" + ctype + ">(" + std::to_string(length) + ");\n";
      fGC += ctype + " * tensor_" + i.first + " = fTensor_" + i.first + ".data();\n";
   }
   fGC += "std::vector<char> fIntermediateMemoryPool = std::vector<char>(" + std::to_string(fArenaBytes) + ");\n";
   for (auto &it : fIntermediateTensorInfos)
      fGC += ConvertTypeToString(it.second.type) + " * tensor_" + it.first + " = nullptr;\n";
   for (size_t id = 0; id < fOperators.size(); id++) fGC += fOperators[id]->GenerateHostSessionMembersCode(std::to_string(id));
   fGC += "\n";
   fGC += "Session(std::string filename =\"" +
          (fUseWeightFile ? fName + (fWeightFile == WeightFileType::Binary ? ".bin" : ".dat") : std::string("")) + "\") {\n";
   for (auto &it : fIntermediateTensorInfos) {
      if (fViewOf.count(it.first)) continue;
      fGC += "   tensor_" + it.first + " = reinterpret_cast<" + ConvertTypeToString(it.second.type) +
             "*>(fIntermediateMemoryPool.data() + " + std::to_string(fPlacement[it.first].offset) + ");\n";
   }
   for (auto &op : fOperators)
      for (auto &out : op->GetOpOutputTensors()) {
         auto v = fViewOf.find(out);
         if (v == fViewOf.end()) continue;
         fGC += "   tensor_" + out + " = reinterpret_cast<" + ConvertTypeToString(fIntermediateTensorInfos[out].type) +
                "*>(tensor_" + v->second + ");\n";
      }
   bool anyWeight = false;
   for (auto &i : fInitializedTensors) anyWeight |= i.second.IsWeightTensor();
   if (fUseWeightFile && anyWeight) {
      fGC += "   std::ifstream f;\n";
      fGC += "   f.open(filename, std::ios::binary);\n";
      fGC += "   if (!f.is_open()) {\n";
      fGC += "      throw std::runtime_error(\"tmva-sofie failed to open file \" + filename + \" for input weights\");\n";
      fGC += "   }\n";
      fGC += "   const bool binary = IsBinaryWeightFile(f);\n";
      for (auto &i : fInitializedTensors) {
         if (!i.second.IsWeightTensor()) continue;
         const std::string tensor_name = "tensor_" + i.first;
         fGC += "   ReadTensor(f, binary, \"" + tensor_name + "\", " + std::to_string(ConvertShapeToLength(i.second.shape())) + ", " +
                std::to_string(static_cast<int>(i.second.type())) + ", " + tensor_name + ");\n";
      }
      fGC += "   f.close();\n";
   } else {
      fGC += "   (void)filename;   // no weight file is read\n";
      for (auto &i : fInitializedTensors) {
         if (!i.second.IsWeightTensor()) continue;
         const size_t length = ConvertShapeToLength(i.second.shape());
         std::stringstream lit;
         lit << "   { static const " << ConvertTypeToString(i.second.type()) << " host[" << (length ? length : 1) << "] = {";
         for (size_t idx = 0; idx < length; ++idx) {
            if (idx) lit << ", ";
            if (i.second.type() == ETensorType::FLOAT) {
               if (!std::isfinite(i.second.data<float>()[idx]))
                  throw std::runtime_error("tmva-sofie tensor_" + i.first + " holds a non-finite value");
               std::stringstream one;
               one << std::setprecision(std::numeric_limits<float>::max_digits10) << i.second.data<float>()[idx];
               std::string text = one.str();
               if (text.find_first_of(".e") == std::string::npos) text += ".";
               lit << text << "f";
            } else {
               switch (i.second.type()) {
               case ETensorType::INT8: lit << (int)i.second.data<int8_t>()[idx]; break;
               case ETensorType::UINT8: lit << (int)i.second.data<uint8_t>()[idx]; break;
               case ETensorType::INT32: lit << i.second.data<int32_t>()[idx]; break;
               case ETensorType::INT64: lit << i.second.data<int64_t>()[idx]; break;
               default: throw std::runtime_error("tmva-sofie tensor_" + i.first + " cannot be written as a literal");
               }
            }
         }
         lit << "};\n     std::copy(host, host + " << length << ", tensor_" << i.first << "); }\n";
         fGC += lit.str();
      }
   }
   for (size_t id = 0; id < fOperators.size(); id++) fGC += fOperators[id]->GenerateHostInitCode(std::to_string(id));
   fGC += "}\n\n";

   // ---- infer: the reference's signature and return convention (RModel.cxx:680-801)
   const size_t nout = fOutputTensorNames.size();
   if (nout == 0) throw std::runtime_error("TMVA-SOFIE: output size=0 are not supported");
   const std::string out = fOutputTensorNames[0];
   const std::string otype = ConvertTypeToString(GetTensorType(out));
   bool sameOutputTypes = true;
   for (auto &n : fOutputTensorNames) sameOutputTypes = sameOutputTypes && GetTensorType(n) == GetTensorType(out);
   std::string inferReturnType = "std::vector<" + otype + ">";
   if (nout > 1) {
      if (sameOutputTypes) {
         inferReturnType = "std::vector<std::vector<" + otype + ">>";
      } else {
         inferReturnType = "std::tuple<";
         for (size_t i = 0; i < nout; ++i)
            inferReturnType += std::string(i ? "," : "") + "std::vector<" + ConvertTypeToString(GetTensorType(fOutputTensorNames[i])) + ">";
         inferReturnType += ">";
      }
   }
   auto outputCount = [&](const std::string &n) {
      const size_t len = ConvertShapeToLength(GetTensorShape(n));
      return (fRuntimeBatch && fBatchTensors.count(n)) ? "fBatch * " + std::to_string(len / fBatchCapacity) : std::to_string(len);
   };
   auto body = [&]() {
      for (size_t id = 0; id < fOperators.size(); id++) {
         if (fOperators[id]->IsFusedAway() || fOperators[id]->IsAbsorbed()) continue;
         fGC += fOperators[id]->GenerateHost(std::to_string(id));
      }
      if (nout == 1) {
         fGC += "   return std::vector<" + otype + ">(tensor_" + out + ", tensor_" + out + " + " + outputCount(out) + ");\n";
         return;
      }
      fGC += "   return " + inferReturnType + "{";
      for (size_t i = 0; i < nout; ++i) {
         const std::string &n = fOutputTensorNames[i];
         fGC += std::string(i ? ", " : "") + "std::vector<" + ConvertTypeToString(GetTensorType(n)) + ">(tensor_" + n + ", tensor_" + n +
                " + " + outputCount(n) + ")";
      }
      fGC += "};\n";
   };
   if (fRuntimeBatch) {
      fGC += inferReturnType + " infer(size_t batch, " + GenerateInferSignature(true) + "){\n";
      fGC += "   if (batch == 0 || batch > " + std::to_string(fBatchCapacity) +
             ") throw std::runtime_error(\"TMVA SOFIE: the batch must be between 1 and " + std::to_string(fBatchCapacity) +
             ", the size this Session was generated for\");\n";
      fGC += "   fBatch = batch;\n";
      body();
      fGC += "}\n";
      fGC += inferReturnType + " infer(" + GenerateInferSignature(true) + "){ return infer(" + std::to_string(fBatchCapacity) + ", " +
             GenerateInferSignature(false) + "); }\n";
   } else {
      fGC += inferReturnType + " infer(" + GenerateInferSignature(true) + "){\n";
      body();
      fGC += "}\n";
   }
   fGC += "};\n";
}

void RModel::Generate(std::underlying_type_t<Options> options, int batchSize, long pos, bool verbose)
{
   fVerbose = verbose;
   // Options::kNoSession (RModel.cxx:1164-1180 of the reference: free function infer, weights as literals). Device
   // weights and buffers still need an owner: the Session is emitted as usual, without a weight file, and the free
   // functions behind it run on one instance created at their first call.
   const bool noSession = (static_cast<std::underlying_type_t<Options>>(Options::kNoSession) & options) != 0;
   if (noSession) {
      fUseWeightFile = false;
      fWeightFile = WeightFileType::None;
   }
   if (static_cast<std::underlying_type_t<Options>>(Options::kRootBinaryWeightFile) & options)
      throw std::runtime_error("TMVA-SOFIE: ROOT binary weight files are not available in this build");
   if (static_cast<std::underlying_type_t<Options>>(Options::kNoWeightFile) & options) {
      fUseWeightFile = false;
      fWeightFile = WeightFileType::None;
   } else if (static_cast<std::underlying_type_t<Options>>(Options::kBinaryWeightFile) & options) {
      fWeightFile = WeightFileType::Binary;
   }
   (void)pos;
   fRuntimeBatch = (static_cast<std::underlying_type_t<Options>>(Options::kRuntimeBatch) & options) != 0;
   if (fRuntimeBatch && batchSize <= 0)
      throw std::runtime_error("TMVA-SOFIE: Options::kRuntimeBatch needs the largest batch as the batch size given to Generate");
   fHostCode = (static_cast<std::underlying_type_t<Options>>(Options::kHostCode) & options) != 0;
   Initialize(batchSize, verbose);
   if (fHostCode) {
      // every operator emits its own statements, as in the reference. Of the fusion passes only the one that hands a
      // Relu to the operator in front of it runs: the operator then ends in the ReLU loop (Gemm, Conv) or, for a
      // quantized operator, clamps at its output zero-point, which a Relu operator on its own does not know
      FuseActivations();
      PlanIntermediateMemory();
      fGC.clear();
      std::string hostGuard;
      GenerateHostHeaderInfo(hostGuard);
      GenerateHostSessionCode();
      if (noSession) {
         fGC += "\n// Options::kNoSession: free function infer on one Session created at the first call\n";
         fGC += "inline Session& DefaultSession() { static Session session(\"\"); return session; }\n";
         fGC += "inline auto infer(" + GenerateInferSignature(true) + "){ return DefaultSession().infer(" + GenerateInferSignature(false) + "); }\n";
      }
      fGC += ("} //SOFIE_" + fName + "\n");
      fGC += "\n#endif  // " + hostGuard + "\n";
      return;
   }
   FuseBatchNorm();
   FuseActivations();
   if (!(static_cast<std::underlying_type_t<Options>>(Options::kLayerPerCall) & options)) {
      FuseGemmChain();
      FuseQLinearPair();
   }
   FusePooling();
   FuseInputQuantization();
   if (!(static_cast<std::underlying_type_t<Options>>(Options::kLayerPerCall) & options)) FuseQLinearConvChain();
   PlanIntermediateMemory();
   fGC.clear();
   std::string hgname;
   GenerateHeaderInfo(hgname);
   GenerateSessionCode();
   if (noSession) {
      fGC += "\n// Options::kNoSession: free functions on one Session that is created at the first call (not re-entrant,\n";
      fGC += "// as the reference's free infer with its static buffers)\n";
      fGC += "inline Session& DefaultSession() { static Session session(\"\"); return session; }\n";
      fGC += "inline auto infer(" + GenerateInferSignature(true) + "){ return DefaultSession().infer(" + GenerateInferSignature(false) + "); }\n";
      if (fRuntimeBatch)
         fGC += "inline auto infer(size_t batch, " + GenerateInferSignature(true) + "){ return DefaultSession().infer(batch, " +
                GenerateInferSignature(false) + "); }\n";
   }
   fGC += ("} //SOFIE_" + fName + "\n");
   fGC += "\n#endif  // " + hgname + "\n";
}

void RModel::PrintGenerated() { std::cout << fGC; }

void RModel::OutputGenerated(std::string filename, bool append)
{
   if (filename == "") filename = fName + ".hxx";
   std::ofstream f;
   f.open(filename, append ? std::ios::app : std::ios::out);
   if (!f.is_open()) throw std::runtime_error("tmva-sofie failed to open file for output generated inference code");
   f << fGC;
   f.close();
   if (fUseWeightFile) {
      // weight file next to the header, same stem (RModel.cxx:1290-1310)
      size_t p = filename.find(".hxx");
      std::string dat = filename;
      const bool binary = fWeightFile == WeightFileType::Binary;
      if (p != std::string::npos) dat.replace(p, 4, binary ? ".bin" : ".dat");
      else dat += binary ? ".bin" : ".dat";
      if (binary) WriteInitializedTensorsToBinaryFile(dat);
      else WriteInitializedTensorsToFile(dat);
   }
}

}   // namespace SOFIE
