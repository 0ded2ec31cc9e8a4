// BatchNormalization emitter (inference). Constructor, checks and error messages follow the reference's
// ROperator_BatchNormalization<T> (src/SOFIE_core/inc/SOFIE/ROperator_BatchNormalization.hxx:41-60,83-126);
// like the reference's Initialize (:127-192) the variance is folded into the scale at generation time,
// scale'[c] = scale[c] * float(1. / sqrt(var[c] + epsilon)), but the result stays one value per channel:
// the kernel broadcasts, where the reference materialises four tensors of the input's shape.
// Emitted code: one sofie_hip_batchnorm_f32 call, y = (x - mean) * scale' + bias, optional ReLU.
// When the operator follows a float Conv that nobody else reads, RModel::FuseBatchNorm folds it into the
// convolution's weights and bias instead (W'[oc] = W[oc] * scale'[oc], b' = (b - mean) * scale' + bias) and
// this operator emits nothing.
#ifndef SOFIE_ROPERATOR_BatchNormalization
#define SOFIE_ROPERATOR_BatchNormalization

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

template <typename T>
class ROperator_BatchNormalization final : public ROperator {
private:
   float fepsilon = 1e-05;
   float fmomentum = 0.9;
   std::size_t ftraining_mode = 0;
   std::string fNX, fNScale, fNB, fNMean, fNVar, fNY, fNFolded;
   EActivationType fActivation;
   std::vector<size_t> fShapeX;
   std::vector<float> fFolded, fMean, fBias;

public:
   ROperator_BatchNormalization() = delete;
   ROperator_BatchNormalization(float epsilon, float momentum, std::size_t training_mode, std::string nameX,
                                std::string nameScale, std::string nameB, std::string nameMean, std::string nameVar,
                                std::string nameY, EActivationType activation = EActivationType::UNDEFINED)
      : fepsilon(epsilon), fmomentum(momentum), ftraining_mode(training_mode), fNX(UTILITY::Clean_name(nameX)),
        fNScale(UTILITY::Clean_name(nameScale)), fNB(UTILITY::Clean_name(nameB)), fNMean(UTILITY::Clean_name(nameMean)),
        fNVar(UTILITY::Clean_name(nameVar)), fNY(UTILITY::Clean_name(nameY)), fActivation(activation)
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      if (!std::is_same<T, float>::value)
         throw std::runtime_error("TMVA SOFIE Encountered unsupported type parsing a BatchNormalization operator");
   }

   std::string Kind() const override { return "BatchNormalization"; }
   bool FuseActivation(EActivationType act) override
   {
      if (act != EActivationType::RELU || fActivation != EActivationType::UNDEFINED) return false;
      fActivation = act;
      return true;
   }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return {input[0]}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      if (input.size() != 5) throw std::runtime_error("TMVA SOFIE BatchNormalization Op Shape inference need 5 input tensors");
      return input;
   }

   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE BatchNormalization op Input Tensor " + fNX + " fnx is not found in model");
      if (!model.CheckIfTensorAlreadyExist(fNScale))
         throw std::runtime_error("TMVA SOFIE BatchNormalization op Input Tensor " + fNScale + " fns is not found in model");
      if (!model.CheckIfTensorAlreadyExist(fNB))
         throw std::runtime_error("TMVA SOFIE BatchNormalization op Input Tensor " + fNB + " fnb is not found in model");
      if (!model.CheckIfTensorAlreadyExist(fNMean))
         throw std::runtime_error("TMVA SOFIE BatchNormalization op Input Tensor " + fNMean + " fnm is not found in model");
      if (!model.CheckIfTensorAlreadyExist(fNVar))
         throw std::runtime_error("TMVA SOFIE BatchNormalization op Input Tensor " + fNVar + " fnv is not found in model");
      if (ftraining_mode != 0)
         throw std::runtime_error("TMVA SOFIE BatchNormalization Op: training mode is not supported");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() < 2 || fShapeX.size() > 4)
         throw std::runtime_error("TMVA SOFIE BatchNormalization Op input tensor " + fNX + " fnx has wrong shape : " +
                                  ConvertShapeToString(fShapeX));
      const size_t channels = fShapeX[1];
      for (auto *name : {&fNScale, &fNB, &fNMean, &fNVar}) {
         if (!model.IsInitializedTensor(*name) || model.GetTensorType(*name) != ETensorType::FLOAT ||
             ConvertShapeToLength(model.GetTensorShape(*name)) != channels)
            throw std::runtime_error("TMVA SOFIE BatchNormalization Op: " + *name +
                                     " must be a float initializer with one value per channel");
      }
      const float *scale = static_cast<float *>(model.GetInitializedTensorData(fNScale).get());
      const float *bias = static_cast<float *>(model.GetInitializedTensorData(fNB).get());
      const float *mean = static_cast<float *>(model.GetInitializedTensorData(fNMean).get());
      const float *var = static_cast<float *>(model.GetInitializedTensorData(fNVar).get());
      fFolded.resize(channels);
      for (size_t c = 0; c < channels; ++c) {
         const float inv = 1. / sqrt(var[c] + fepsilon);
         fFolded[c] = scale[c] * inv;
      }
      fMean.assign(mean, mean + channels);
      fBias.assign(bias, bias + channels);
      fNFolded = fNY + "_bnscale";
      std::shared_ptr<void> data(malloc(channels * sizeof(float)), free);
      std::memcpy(data.get(), fFolded.data(), channels * sizeof(float));
      model.AddInitializedTensor(fNFolded, ETensorType::FLOAT, {channels}, data);
      // gamma and the variance live on in the folded scale only
      model.SetNotWritableInitializedTensor(fNScale);
      model.SetNotWritableInitializedTensor(fNVar);
      fInputTensorNames = {fNX, fNFolded, fNMean, fNB};
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNX), fShapeX);
   }

   // values a preceding convolution needs to absorb this operator
   const std::vector<float> &FoldedScale() const { return fFolded; }
   const std::vector<float> &Mean() const { return fMean; }
   const std::vector<float> &Bias() const { return fBias; }
   bool HasActivation() const { return fActivation == EActivationType::RELU; }
   // initializers that only this operator read: not written or uploaded once it is absorbed
   std::vector<std::string> OwnInitializers() const { return {fNFolded, fNMean, fNB}; }

   std::string Generate(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty())
         throw std::runtime_error("TMVA SOFIE Batch Normalization called to Generate without being initialized first");
      size_t plane = 1;
      for (size_t i = 2; i < fShapeX.size(); ++i) plane *= fShapeX[i];
      std::stringstream out;
      out << "\n\n//---- BatchNorm " << OpName << "\n";
      out << SP << "Check(sofie_hip_batchnorm_f32(fCtx, tensor_" << fNX << ", tensor_" << fNFolded << ", tensor_" << fNMean
          << ", tensor_" << fNB << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0]) << ", " << fShapeX[1] << ", " << plane << ", "
          << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << "), \"BatchNorm " << OpName
          << "\");\n";
      return out.str();
   }

   // host form: the loop of the reference (ROperator_BatchNormalization.hxx Generate: x - mean, times the folded scale,
   // plus the bias, then the ReLU), one rounding per step
   std::string GenerateHost(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty())
         throw std::runtime_error("TMVA SOFIE Batch Normalization called to Generate without being initialized first");
      size_t plane = 1;
      for (size_t i = 2; i < fShapeX.size(); ++i) plane *= fShapeX[i];
      std::stringstream out;
      out << "\n\n//---- BatchNorm " << OpName << "\n";
      out << SP << "for (size_t n = 0; n < " << BatchCount(fShapeX[0]) << "; n++)\n";
      out << SP << SP << "for (size_t c = 0; c < " << fShapeX[1] << "; c++)\n";
      out << SP << SP << SP << "for (size_t i = 0; i < " << plane << "; i++) {\n";
      out << SP << SP << SP << SP << "const size_t id = (n * " << fShapeX[1] << " + c) * " << plane << " + i;\n";
      out << SP << SP << SP << SP << "float v = tensor_" << fNX << "[id] - tensor_" << fNMean << "[c];\n";
      out << SP << SP << SP << SP << "v = v * tensor_" << fNFolded << "[c];\n";
      out << SP << SP << SP << SP << "v = v + tensor_" << fNB << "[c];\n";
      if (fActivation == EActivationType::RELU) out << SP << SP << SP << SP << "v = v > 0 ? v : 0;\n";
      out << SP << SP << SP << SP << "tensor_" << fNY << "[id] = v;\n";
      out << SP << SP << SP << "}\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
