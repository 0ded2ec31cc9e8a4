// Emitter interface: one ROperator per graph node. Same virtuals, call order and naming as
// the reference's src/SOFIE_core/inc/SOFIE/ROperator.hxx:17-57; RModel calls
// Initialize(model) once, then GenerateSessionMembersCode / GenerateInitCode while it writes
// the Session, then Generate(opName) inside infer. The extra hooks at the bottom exist for
// the device emission only (activation fusion, view outputs, constructor-time weight work).
#ifndef SOFIE_ROPERATOR
#define SOFIE_ROPERATOR

#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "SOFIE/SOFIE_common.hxx"

namespace SOFIE {

class RModel;

class ROperator {
public:
   virtual std::vector<std::string> GetBlasRoutines() { return {}; }
   virtual std::vector<std::string> GetStdLibs() { return {}; }
   virtual std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>>) = 0;
   virtual std::vector<ETensorType> TypeInference(std::vector<ETensorType>) = 0;
   virtual void Initialize(RModel &) = 0;
   virtual std::string Generate(std::string OpName) = 0;   // expects a unique OpName per operator
   virtual std::string GenerateInitCode() { return ""; }
   virtual std::string GenerateDeclCode() { return ""; }
   virtual std::string GenerateSessionMembersCode(std::string /*opName*/) { return ""; }
   virtual std::string Header() { return ""; }
   virtual ~ROperator() {}

   // --- device-emission hooks ------------------------------------------------------------
   // operator family name ("Gemm", "Conv", "Relu", ...), used by RModel's fusion pass
   virtual std::string Kind() const { return ""; }
   // try to absorb a following activation into this operator's epilogue
   virtual bool FuseActivation(EActivationType) { return false; }
   // the output is a view of this input tensor (no kernel, no memory): "" if not a view
   virtual std::string ViewOf() const { return ""; }
   // when fused away, the operator emits nothing and its output aliases its input
   void SetFusedAway() { fFusedAway = true; }
   bool IsFusedAway() const { return fFusedAway; }
   // try to absorb a following max pooling (kernel, strides, no pads) whose output tensor becomes this
   // operator's output; on success the operator no longer writes its original output tensor
   virtual bool FusePooling(const std::vector<size_t> & /*kernel*/, const std::vector<size_t> & /*strides*/,
                            const std::string & /*pooledName*/, const std::vector<size_t> & /*pooledShape*/)
   {
      return false;
   }
   // try to absorb a preceding QuantizeLinear (float tensor xFloat quantized with scale / zeroPoint into this
   // operator's int8 input): on success the operator reads the float tensor itself
   virtual bool FuseInputQuantization(const std::string & /*xFloat*/, float /*scale*/, int /*zeroPoint*/) { return false; }
   // try to absorb a following BatchNormalization y = (x - mean[c]) * scale[c] + bias[c] (one value per output
   // channel, the variance already folded into scale) and, if relu is set, the ReLU behind it; on success the
   // operator writes the tensor outName instead of its own output
   virtual bool FuseBatchNorm(RModel & /*model*/, const std::vector<float> & /*scale*/, const std::vector<float> & /*mean*/,
                              const std::vector<float> & /*bias*/, const std::string & /*outName*/, bool /*relu*/)
   {
      return false;
   }
   // Run-time batch: the leading dimension of this operator's first input is the batch, which the generated
   // Session keeps in the member named `expr` (at most `capacity`, the value the shapes were resolved with).
   // Returns false if the operator cannot run on fewer rows than it was generated for.
   virtual bool SetRuntimeBatch(const std::string &expr, size_t capacity)
   {
      fBatchExpr = expr;
      fBatchCapacity = capacity;
      return true;
   }
   // --- host emission (Options::kHostCode) ----------------------------------------------------
   // The operator as code for the host cores, in the reference's way (BLAS::sgemm_ / saxpy_ calls and plain
   // loops on host pointers named tensor_<name>): members of the Session, statements of its constructor, and the
   // statements of infer. An operator without a host form says so when it is asked for one.
   virtual std::string GenerateHost(std::string /*opName*/)
   {
      throw std::runtime_error("TMVA SOFIE " + (Kind().empty() ? std::string("operator") : Kind()) +
                               " Op has no host emission (Options::kHostCode)");
   }
   virtual std::string GenerateHostSessionMembersCode(std::string /*opName*/) { return ""; }
   virtual std::string GenerateHostInitCode(std::string /*opName*/) { return ""; }
   // absorbed into another operator: emits nothing, and its output is written by the absorbing operator
   void SetAbsorbed() { fAbsorbed = true; }
   bool IsAbsorbed() const { return fAbsorbed; }

   const std::vector<std::string> &GetOpInputTensors() const { return fInputTensorNames; }
   const std::vector<std::string> &GetOpOutputTensors() const { return fOutputTensorNames; }

protected:
   const std::string SP = "   ";   // indentation of generated code
   std::string fBatchExpr;         // empty: every dimension is a constant of the generated code
   size_t fBatchCapacity = 0;
   // a count proportional to the batch (rows, images, elements of a batch-led tensor) as emitted text
   std::string BatchCount(size_t value) const
   {
      if (fBatchExpr.empty() || fBatchCapacity == 0) return std::to_string(value);
      if (value % fBatchCapacity != 0)
         throw std::runtime_error("TMVA SOFIE run-time batch: a count of " + std::to_string(value) + " is not a multiple of the batch");
      const size_t per = value / fBatchCapacity;
      return per == 1 ? fBatchExpr : "(" + fBatchExpr + " * " + std::to_string(per) + ")";
   }
   bool fUseSession = false;
   bool fIsOutputConstant = false;
   bool fFusedAway = false;
   bool fAbsorbed = false;
   std::vector<std::string> fInputTensorNames;    // every tensor the emitted code reads
   std::vector<std::string> fOutputTensorNames;   // tensors the emitted code writes
};

}   // namespace SOFIE
#endif
