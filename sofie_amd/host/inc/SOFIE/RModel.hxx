// Graph IR and code-generation driver. Public surface follows the reference's
// src/SOFIE_core/inc/SOFIE/RModel.hxx:61-180 and RModel_Base.hxx:21-90 (AddInputTensorInfo,
// AddInitializedTensor, AddOperator, AddOutputTensorNameList, Generate, OutputGenerated, the
// tensor queries operators use from Initialize). What Generate emits differs: a Session that
// owns a sofie_hip context, device-resident weights (uploaded once in the constructor) and
// one device arena for all intermediates, and whose infer() is a sequence of calls into the
// C ABI of include/sofie_hip.h (one H2D of the input, kernels on one stream, one D2H).
#ifndef SOFIE_RMODEL
#define SOFIE_RMODEL

#include <map>
#include <memory>
#include <set>
#include <string>
#include <type_traits>
#include <unordered_set>
#include <vector>

#include "SOFIE/ROperator.hxx"
#include "SOFIE/SOFIE_common.hxx"

namespace SOFIE {

enum class Options {
   kDefault = 0x0,
   kNoSession = 0x1,             // free function infer on one Session created at its first call; weights as literals
   kNoWeightFile = 0x2,          // weights as literals in the generated header
   kRootBinaryWeightFile = 0x4,  // not available (no ROOT)
   kGNN = 0x8,
   kGNNComponent = 0x10,
   kBinaryWeightFile = 0x20,     // typed binary records in <name>.bin instead of the text <name>.dat (not in the reference)
   kRuntimeBatch = 0x40,         // the batch size given to Generate is a capacity: infer(n, ...) runs any n up to it
   kLayerPerCall = 0x80,         // no chains of fully connected layers in one launch: every Gemm emits its own call
   kHostCode = 0x100,            // code for the host cores, as the reference emits it (BLAS::sgemm_ / saxpy_ and loops on host
                                 // memory) instead of calls into the kernel library: fp32 Gemm, Conv, Relu, pooling, Reshape
};
std::underlying_type_t<Options> operator|(Options opA, Options opB);
std::underlying_type_t<Options> operator|(std::underlying_type_t<Options> opA, Options opB);

enum class WeightFileType { None, RootBinary, Text, Binary };

class RModel {
public:
   RModel() = default;
   RModel(std::string name, std::string parsedtime);
   RModel(RModel &&) = default;
   RModel &operator=(RModel &&) = default;
   RModel(const RModel &) = delete;
   RModel &operator=(const RModel &) = delete;

   int Verbose() const { return fVerbose; }
   bool UseSession() const { return fUseSession; }

   const std::vector<size_t> &GetTensorShape(std::string name) const;
   std::vector<Dim> GetDynamicTensorShape(std::string name) const;
   const ETensorType &GetTensorType(std::string name) const;
   bool CheckIfTensorAlreadyExist(std::string tensor_name);
   bool IsInitializedTensor(const std::string &name) const;
   bool IsDynamicTensor(const std::string &) const { return false; }
   bool IsDimInputTensor(const std::string &) const { return false; }
   bool IsReadyInputTensor(const std::string &name) const;

   void AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<Dim> shape);
   void AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<size_t> shape);
   void AddInputTensorName(std::string name);
   void AddOperator(std::unique_ptr<ROperator> op, int order_execution = -1);
   void AddOperatorReference(ROperator *op, int order_execution = -1)
   {
      AddOperator(std::unique_ptr<ROperator>(op), order_execution);
   }
   void AddInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape,
                             std::shared_ptr<void> data);
   template <typename T>
   void AddInitializedTensor(const std::string &tensor_name, const std::vector<std::size_t> &shape, T *raw_data)
   {
      size_t size = ConvertShapeToLength(shape);
      std::shared_ptr<void> data(malloc(size * sizeof(T)), free);
      std::memcpy(data.get(), raw_data, size * sizeof(T));
      AddInitializedTensor(tensor_name, GetTemplatedType(T()), shape, data);
   }
   void UpdateInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape,
                                std::shared_ptr<void> data);
   std::shared_ptr<void> GetInitializedTensorData(std::string tensor_name);
   void SetNotWritableInitializedTensor(const std::string &tensor_name);
   // Channels-last bookkeeping of int8 activations. The quantized operators keep 4-D activations as
   // [N,H,W,C] in memory (the order the matrix-core convolution reads); the tensor's shape stays the
   // logical [N,C,H,W]. A Flatten of such a tensor is recorded with the same (C,H,W) so that the next
   // matrix product can permute its weight rows instead of moving the activations.
   void MarkChannelsLast(const std::string &name, size_t C, size_t H, size_t W) { fChannelsLast[name] = {C, H, W}; }
   bool IsChannelsLast(const std::string &name, std::vector<size_t> *chw = nullptr) const
   {
      auto it = fChannelsLast.find(name);
      if (it == fChannelsLast.end()) return false;
      if (chw) *chw = it->second;
      return true;
   }
   void AddIntermediateTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape);
   void AddIntermediateTensor(std::string tensor_name, ETensorType type, std::vector<Dim> dim_shape);
   void AddOutputTensorNameList(std::vector<std::string> output_tensor_names);

   void AddBlasRoutines(std::vector<std::string> routines);
   void AddNeededStdLib(std::string libname);
   void AddNeededCustomHeader(std::string filename) { fCustomOpHeaders.insert(filename); }

   void Initialize(int batchSize = -1, bool verbose = false);
   void Initialize(const std::map<std::string, size_t> &inputParams, bool verbose = false);
   void Generate(std::underlying_type_t<Options> options, int batchSize = -1, long pos = 0, bool verbose = false);
   void Generate(Options options = Options::kDefault, int batchSize = -1, int pos = 0, bool verbose = false)
   {
      Generate(static_cast<std::underlying_type_t<Options>>(options), batchSize, pos, verbose);
   }
   std::string GenerateInferSignature(bool isdecl = true);

   void PrintGenerated();
   std::string ReturnGenerated() { return fGC; }
   void OutputGenerated(std::string filename = "", bool append = false);
   long WriteInitializedTensorsToFile(std::string filename = "");
   long WriteInitializedTensorsToBinaryFile(std::string filename = "");
   std::string GenerateWeightReaderHelpers();
   void ReadInitializedTensorsFromFile(long pos);

   const std::vector<std::string> &GetInputTensorNames() const { return fInputTensorNames; }
   const std::vector<std::string> &GetOutputTensorNames() const { return fOutputTensorNames; }
   void SetFilename(std::string filename) { fName = filename; }
   std::string GetFilename() { return fName; }
   const std::string &GetName() const { return fName; }
   // total bytes of the device arena after Generate (0 before)
   size_t GetIntermediateMemorySize() const { return fArenaBytes; }

private:
   struct Placement {
      size_t offset = 0, bytes = 0;
      int first = 0, last = 0;
   };
   void FuseBatchNorm();
   void FuseGemmChain();
   void FuseQLinearPair();
   void FuseActivations();
   void FusePooling();
   void FuseInputQuantization();
   void FuseQLinearConvChain();
   void PlanIntermediateMemory();
   void GenerateHeaderInfo(std::string &hgname);
   void GenerateSessionCode();
   void GenerateHostHeaderInfo(std::string &hgname);
   void GenerateHostSessionCode();
   std::string RootOf(const std::string &name) const;

   std::string fFileName, fParseTime, fName = "UnnamedModel", fGC;
   WeightFileType fWeightFile = WeightFileType::Text;
   bool fUseWeightFile = true, fUseSession = true, fIsInitialized = false, fHostCode = false;
   int fVerbose = 0;

   std::map<std::string, TensorInfo> fReadyInputTensorInfos;
   struct ParametricInput { ETensorType type; std::vector<Dim> shape; };
   std::map<std::string, ParametricInput> fInputTensorInfos;   // inputs whose shape still holds a parameter
   std::map<std::string, InitializedTensor> fInitializedTensors;
   std::map<std::string, TensorInfo> fIntermediateTensorInfos;
   std::vector<std::string> fOutputTensorNames, fInputTensorNames;
   std::vector<std::unique_ptr<ROperator>> fOperators;
   std::unordered_set<std::string> fNeededBlasRoutines, fCustomOpHeaders;
   std::set<std::string> fNeededStdLib = {"vector"};
   const std::set<std::string> fAllowedStdLib = {"vector", "algorithm", "cmath", "memory", "span"};

   // Options::kRuntimeBatch: tensors whose leading dimension is the batch parameter, and the value it was resolved with
   bool fRuntimeBatch = false;
   size_t fBatchCapacity = 0;
   std::set<std::string> fBatchTensors;
   std::map<std::string, std::string> fViewOf;      // view tensor -> tensor it aliases
   std::map<std::string, std::vector<size_t>> fChannelsLast;   // tensor stored channels-last -> (C,H,W)
   std::map<std::string, Placement> fPlacement;     // arena slot of every non-view intermediate
   size_t fArenaBytes = 0;
   const std::string SP = "   ";
};

}   // namespace SOFIE
#endif
