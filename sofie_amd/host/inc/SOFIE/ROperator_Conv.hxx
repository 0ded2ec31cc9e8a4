// Conv emitter (2-D). Constructor, attribute defaults, output-shape rule and error messages follow the
// reference's ROperator_Conv<T> (src/SOFIE_core/inc/SOFIE/ROperator_Conv.hxx:52-87,95-201,203-282):
//   - auto_pad NOTSET with no pads attribute means 1 on every side (:136-139, not ONNX's 0);
//   - SAME_UPPER / SAME_LOWER start from k/2 and add one at the begin / end for odd kernels (:140-158);
//   - begin/end pads that differ are averaged with a warning (:387-401);
//   - group == 0 means C / C_w (:110-112).
// Emitted code: one sofie_hip_conv2d_f32 call over the whole batch (implicit GEMM, bias and
// optional ReLU fused) instead of the per-image weight re-layout + Im2col + sgemm_ + saxpy_.
#ifndef SOFIE_SOFIE_ROPERATOR_CONV
#define SOFIE_SOFIE_ROPERATOR_CONV

#include <cstdlib>
#include <iostream>
#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

// Attribute handling shared by Conv and QLinearConv.
struct ConvGeometry {
   std::string autopad;
   std::vector<size_t> dilations, kernel, pads, strides;
   size_t group = 0;
   // fills defaults, returns the output shape [N, OC, OH, OW] for input [N,C,H,W] and weights [OC,C/g,KH,KW]
   std::vector<size_t> Resolve(const std::vector<size_t> &x, const std::vector<size_t> &w)
   {
      if (x.size() != 4 || w.size() != 4)
         throw std::runtime_error("TMVA SOFIE Conv Op: only 2-D convolutions (4-D tensors) are supported by the device emission");
      if (group == 0) group = x[1] / w[1];
      size_t k1 = kernel.empty() ? w[2] : kernel[0];
      size_t k2 = kernel.empty() ? w[3] : kernel[1];
      if (dilations.empty()) dilations = {1, 1};
      dilations.resize(2, 1);
      // dilated extent of the kernel
      const size_t e1 = k1 + (dilations[0] - 1) * (k1 - 1), e2 = k2 + (dilations[1] - 1) * (k2 - 1);
      kernel = {k1, k2};
      if (autopad == "NOTSET" || autopad == "") {
         if (pads.empty()) pads = {1, 1, 1, 1};
      } else if (autopad == "SAME_UPPER" || autopad == "SAME_LOWER") {
         pads = {e1 / 2, e2 / 2, e1 / 2, e2 / 2};
         if (e1 % 2 == 1) (autopad == "SAME_UPPER") ? pads[0]++ : pads[2]++;
         if (e2 % 2 == 1) (autopad == "SAME_UPPER") ? pads[1]++ : pads[3]++;
      } else if (autopad == "VALID") {
         pads = {0, 0, 0, 0};
      } else {
         throw std::runtime_error("TMVA SOFIE Conv Op invalid fAutopad");
      }
      pads.resize(4, 0);
      if (strides.empty()) strides = {1, 1};
      strides.resize(2, 1);
      const size_t oh = (x[2] + pads[0] + pads[2] - e1) / strides[0] + 1;
      const size_t ow = (x[3] + pads[1] + pads[3] - e2) / strides[1] + 1;
      return {x[0], w[0], oh, ow};
   }
   // symmetric pads handed to the kernel
   void SymmetricPads(size_t &ph, size_t &pw)
   {
      if (pads[0] != pads[2] || pads[1] != pads[3]) {
         std::cout << "TMVA SOFIE Operator Conv:  asymmetric padding not supported. Assume an average padding " << std::endl;
         pads[0] = (pads[0] + pads[2]) / 2;
         pads[1] = (pads[1] + pads[3]) / 2;
      }
      ph = pads[0];
      pw = pads[1];
   }
};

template <typename T>
class ROperator_Conv final : public ROperator {
private:
   ConvGeometry fGeom;
   std::string fNX, fNW, fNB, fNY;
   std::vector<size_t> fShapeX, fShapeW, fShapeB, fShapeY;
   EActivationType fActivation = EActivationType::UNDEFINED;

public:
   ROperator_Conv() {}
   ROperator_Conv(std::string autopad, std::vector<size_t> dilations, size_t group, std::vector<size_t> kernelShape,
                  std::vector<size_t> pads, std::vector<size_t> strides, std::string nameX, std::string nameW,
                  std::string nameB, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNW(UTILITY::Clean_name(nameW)), fNB(UTILITY::Clean_name(nameB)),
        fNY(UTILITY::Clean_name(nameY))
   {
      if (!std::is_same<T, float>::value)
         throw std::runtime_error("TMVA SOFIE Encountered unsupported type parsing a Conv operator");
      fGeom.autopad = autopad; fGeom.dilations = dilations; fGeom.group = group; fGeom.kernel = kernelShape;
      fGeom.pads = pads; fGeom.strides = strides;
      fInputTensorNames = {fNX, fNW, fNB};
      fOutputTensorNames = {fNY};
   }
   ROperator_Conv(std::string autopad, std::vector<size_t> dilations, size_t group, std::vector<size_t> kernelShape,
                  std::vector<size_t> pads, std::vector<size_t> strides, std::string nameX, std::string nameW,
                  std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNW(UTILITY::Clean_name(nameW)), fNY(UTILITY::Clean_name(nameY))
   {
      if (!std::is_same<T, float>::value)
         throw std::runtime_error("TMVA SOFIE Encountered unsupported type parsing a Conv operator");
      fGeom.autopad = autopad; fGeom.dilations = dilations; fGeom.group = group; fGeom.kernel = kernelShape;
      fGeom.pads = pads; fGeom.strides = strides;
      fInputTensorNames = {fNX, fNW};
      fOutputTensorNames = {fNY};
   }

   std::string Kind() const override { return "Conv"; }
   bool FuseActivation(EActivationType act) override
   {
      if (act != EActivationType::RELU || fActivation != EActivationType::UNDEFINED) return false;
      fActivation = act;
      return true;
   }
   // Conv -> BatchNormalization: W'[oc] = W[oc] * scale[oc], b'[oc] = (b[oc] - mean[oc]) * scale[oc] + bias[oc],
   // written as new initializers; the convolution then produces the normalised tensor directly.
   bool FuseBatchNorm(RModel &model, const std::vector<float> &scale, const std::vector<float> &mean,
                      const std::vector<float> &bias, const std::string &outName, bool relu) override
   {
      if (fShapeW.empty() || fActivation != EActivationType::UNDEFINED) return false;
      if (!model.IsInitializedTensor(fNW) || (fNB != "" && !model.IsInitializedTensor(fNB))) return false;
      const size_t oc = fShapeW[0];
      if (scale.size() != oc || mean.size() != oc || bias.size() != oc) return false;
      const size_t per = ConvertShapeToLength(fShapeW) / oc;
      const float *w = static_cast<float *>(model.GetInitializedTensorData(fNW).get());
      const float *b = fNB != "" ? static_cast<float *>(model.GetInitializedTensorData(fNB).get()) : nullptr;
      std::shared_ptr<void> nw(malloc(oc * per * sizeof(float)), free), nb(malloc(oc * sizeof(float)), free);
      float *pw = static_cast<float *>(nw.get()), *pb = static_cast<float *>(nb.get());
      for (size_t c = 0; c < oc; ++c) {
         for (size_t i = 0; i < per; ++i) pw[c * per + i] = w[c * per + i] * scale[c];
         pb[c] = ((b ? b[c] : 0.0f) - mean[c]) * scale[c] + bias[c];
      }
      const std::string foldedW = outName + "_bnw", foldedB = outName + "_bnb";
      model.AddInitializedTensor(foldedW, ETensorType::FLOAT, fShapeW, nw);
      model.AddInitializedTensor(foldedB, ETensorType::FLOAT, {oc}, nb);
      fNW = foldedW;
      fNB = foldedB;
      fShapeB = {oc};
      fNY = outName;
      fInputTensorNames = {fNX, fNW, fNB};
      fOutputTensorNames = {fNY};
      if (relu) fActivation = EActivationType::RELU;
      return true;
   }
   const std::string &WeightName() const { return fNW; }
   const std::string &BiasName() const { return fNB; }

   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return {input[0]}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      if (input.size() > 3) throw std::runtime_error("TMVA SOFIE Conv Op Shape inference need 2 or 3 input tensors");
      return {fGeom.Resolve(input[0], input[1])};
   }

   void Initialize(RModel &model) override
   {
      fUseSession = model.UseSession();
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE Conv op Input Tensor " + fNX + " is not found in model");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() != 4)
         throw std::runtime_error("TMVA SOFIE Conv Op input data tensor" + fNX + " is not of 4 dimensions (1-D and 3-D "
                                  "convolutions are not supported by the device emission)");
      if (!model.CheckIfTensorAlreadyExist(fNW))
         throw std::runtime_error("TMVA SOFIE Conv op Input weight Tensor " + fNW + " is not found in model");
      fShapeW = model.GetTensorShape(fNW);
      if (fShapeW.size() != 4)
         throw std::runtime_error("TMVA SOFIE Conv Op input weight tensor" + fNW + " is not of 4 dimensions");
      fShapeY = ShapeInference({fShapeX, fShapeW})[0];
      if (fShapeW[1] * fGeom.group != fShapeX[1])
         throw std::runtime_error("TMVA SOFIE Conv op: weight tensor " + fNW + " does not match the input channels and group");
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNX), fShapeY);
      if (fNB != "") {
         if (!model.CheckIfTensorAlreadyExist(fNB))
            throw std::runtime_error("TMVA SOFIE Conv op Input Tensor " + fNB + " is not found in model");
         fShapeB = model.GetTensorShape(fNB);
         if (fShapeB.size() < 1) throw std::runtime_error("TMVA SOFIE Conv op: Bias Tensor has empty shape");
         // one value per filter; the kernel broadcasts it (the reference materialises [OC,OH,OW], :284-300)
         if (fShapeB[0] != fShapeY[1] || ConvertShapeToLength(fShapeB) != fShapeY[1])
            throw std::runtime_error("TMVA SOFIE Conv op: Bias Tensor has wrong shape: " + ConvertShapeToString(fShapeB));
      }
   }

   std::string Generate(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeW.empty() || (fNB != "" && fShapeB.empty()) || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Conv Op called to Generate without being initialized first");
      size_t ph, pw;
      fGeom.SymmetricPads(ph, pw);
      std::stringstream out;
      out << "\n//----  operator Conv " << OpName << "\n";
      out << SP << "Check(sofie_hip_conv2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNW << ", "
          << (fNB.empty() ? std::string("nullptr") : "tensor_" + fNB) << ", tensor_" << fNY << ", " << fShapeX[0] << ", "
          << fShapeX[1] << ", " << fShapeX[2] << ", " << fShapeX[3] << ", " << fShapeW[0] << ", " << fShapeW[2] << ", "
          << fShapeW[3] << ", " << ph << ", " << pw << ", " << fGeom.strides[0] << ", " << fGeom.strides[1] << ", "
          << fGeom.dilations[0] << ", " << fGeom.dilations[1] << ", " << fGeom.group << ", "
          << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << "), \"Conv " << OpName << "\");\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
