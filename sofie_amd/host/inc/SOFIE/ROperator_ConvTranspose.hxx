// ConvTranspose emitter (1-D and 2-D). Constructor, attribute defaults, output-shape rule and error
// messages follow the reference's ROperator_ConvTranspose<T>
// (src/SOFIE_core/inc/SOFIE/ROperator_ConvTranspose.hxx:64-84, ROperator_ConvTranspose.icc:14-103,106-190):
//   - group 0 means 1; strides, dilations default to 1, output_padding and pads to 0;
//   - output extent = stride*(in-1) + kernel extent + output_padding - pad_begin - pad_end (:83-90), where the
//     kernel extent counts the dilation;
//   - an explicit output_shape attribute and auto_pad other than NOTSET are refused (:52-79,:91-97);
//   - begin/end pads that differ: the reference averages them with a warning at generation time (:318-346) while
//     the declared output extent uses their sum; here both reach the library and the result is ONNX's;
//   - 3-D transposed convolutions are refused (:391).
// Emitted code: one sofie_hip_conv_transpose2d_f32 call over the whole batch (bias and optional ReLU
// fused) instead of the kernel re-layout loop, sgemm_ into a column matrix, col2im and saxpy_ per image.
// A 1-D operator [N,C,W] runs as the 2-D one on [N,C,1,W].
#ifndef SOFIE_SOFIE_ROPERATOR_CONVTRANSPOSE_HXX
#define SOFIE_SOFIE_ROPERATOR_CONVTRANSPOSE_HXX

#include <iostream>
#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

template <typename T>
class ROperator_ConvTranspose final : public ROperator {
private:
   std::string fAttrAutopad;
   std::vector<size_t> fAttrDilations;
   size_t fAttrGroup = 0;
   std::vector<size_t> fAttrKernelShape, fAttrOutputPadding, fAttrOutputShape, fAttrPads, fAttrStrides;
   std::string fNX, fNW, fNB, fNY;
   std::vector<size_t> fShapeX, fShapeW, fShapeB, fShapeY;
   size_t fDim = 0;
   EActivationType fActivation = EActivationType::UNDEFINED;

public:
   ROperator_ConvTranspose() {}
   ROperator_ConvTranspose(std::string autopad, std::vector<size_t> dilations, size_t group, std::vector<size_t> kernelShape,
                           std::vector<size_t> outputPadding, std::vector<size_t> outputShape, std::vector<size_t> pads,
                           std::vector<size_t> strides, std::string nameX, std::string nameW, std::string nameB,
                           std::string nameY)
      : fAttrAutopad(autopad), fAttrDilations(dilations), fAttrGroup(group), fAttrKernelShape(kernelShape),
        fAttrOutputPadding(outputPadding), fAttrOutputShape(outputShape), fAttrPads(pads), fAttrStrides(strides),
        fNX(UTILITY::Clean_name(nameX)), fNW(UTILITY::Clean_name(nameW)), fNB(UTILITY::Clean_name(nameB)),
        fNY(UTILITY::Clean_name(nameY))
   {
      if (!std::is_same<T, float>::value)
         throw std::runtime_error("TMVA SOFIE Encountered unsupported type parsing a Conv operator");
      fInputTensorNames = {fNX, fNW};
      if (!fNB.empty()) fInputTensorNames.emplace_back(fNB);
      fOutputTensorNames = {fNY};
   }

   std::string Kind() const override { return "ConvTranspose"; }
   bool FuseActivation(EActivationType act) override
   {
      if (act != EActivationType::RELU || fActivation != EActivationType::UNDEFINED) return false;
      fActivation = act;
      return true;
   }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return {input[0]}; }

   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      const std::vector<size_t> &inputShape = input[0];
      const std::vector<size_t> &weightShape = input[1];
      const size_t size = inputShape.size();
      fDim = size - 2;
      if (fAttrGroup == 0) fAttrGroup = 1;
      if (fAttrStrides.empty()) fAttrStrides = std::vector<size_t>(fDim, 1);
      if (fAttrDilations.empty()) fAttrDilations = std::vector<size_t>(fDim, 1);
      // kernel extent including the dilation, always taken from the weight tensor (the reference does so only
      // when the kernel_shape attribute is absent, :31-35, and otherwise forgets the dilation)
      fAttrKernelShape.resize(fDim);
      for (size_t i = 0; i < fDim; i++)
         fAttrKernelShape[i] = weightShape[i + 2] + (fAttrDilations[i] - 1) * (weightShape[i + 2] - 1);
      if (fAttrOutputPadding.empty()) fAttrOutputPadding = std::vector<size_t>(fDim, 0);
      std::vector<size_t> outShape(size);
      outShape[0] = inputShape[0];
      outShape[1] = weightShape[1] * fAttrGroup;
      if (fAttrPads.empty()) {
         fAttrPads = std::vector<size_t>(2 * fDim, 0);
         if (fAttrOutputShape.size() == fDim)
            throw std::runtime_error("ConvTranspose with output_shape explicitly set not yet supported.");
         if (fAttrAutopad != "NOTSET" && fAttrAutopad != "")
            throw std::runtime_error("ConvTranspose with padding SAME_UPPER or SMAE_LOWER not supported");
      }
      if (!fAttrOutputShape.empty())
         throw std::runtime_error("ConvTranspose with output_shape explicitly set not yet supported.");
      for (size_t i = 0; i < fDim; i++) {
         const size_t j = i + 2;
         outShape[j] = fAttrStrides[i] * (inputShape[j] - 1) + fAttrKernelShape[i] + fAttrOutputPadding[i] - fAttrPads[i] -
                       fAttrPads[fDim + i];
      }
      return {outShape};
   }

   void Initialize(RModel &model) override
   {
      fUseSession = model.UseSession();
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE Conv Transpose op Input Tensor " + fNX + " is not found in model");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() < 3 || fShapeX.size() > 5)
         throw std::runtime_error("TMVA SOFIE Conv Transpose Op input data tensor" + fNX + " is not of 3,4 or 5 dimensions");
      if (!model.CheckIfTensorAlreadyExist(fNW))
         throw std::runtime_error("TMVA SOFIE Conv op Input weight Tensor " + fNW + " is not found in model");
      fShapeW = model.GetTensorShape(fNW);
      if (fShapeW.size() < 3 || fShapeW.size() > 5 || fShapeW.size() != fShapeX.size())
         throw std::runtime_error("TMVA SOFIE Conv Transpose Op input weight tensor" + fNW + " is not of 3,4 or 5 dimensions");
      if (fShapeX.size() == 5) throw std::runtime_error("TMVA SOFIE 3D Conv Transpose not yet supported");
      fShapeY = ShapeInference({fShapeX, fShapeW})[0];
      if (fShapeW[0] != fShapeX[1] || fShapeX[1] % fAttrGroup != 0)
         throw std::runtime_error("TMVA SOFIE Conv Transpose op: weight tensor " + fNW + " does not match the input channels and group");
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNX), fShapeY);
      if (fNB != "") {
         if (!model.CheckIfTensorAlreadyExist(fNB))
            throw std::runtime_error("TMVA SOFIE ConvTrans op Input Tensor " + fNB + " is not found in model");
         fShapeB = model.GetTensorShape(fNB);
         if (fShapeB.size() < 1) throw std::runtime_error("TMVA SOFIE ConvTrans op: Bias Tensor has empty shape");
         // one value per filter; the kernel broadcasts it (the reference materialises the output shape, :146-170)
         if (ConvertShapeToLength(fShapeB) != fShapeY[1])
            throw std::runtime_error("TMVA SOFIE ConvTrans op: Bias Tensor has wrong shape: " + ConvertShapeToString(fShapeB));
      }
   }

   std::string Generate(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeW.empty() || (fNB != "" && fShapeB.empty()) || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Conv Op called to Generate without being initialized first");
      // the library places the result by the begin pads and is told the output extent (which the end pads shorten):
      // begin and end pads that differ are exact
      const bool oneD = fDim == 1;
      const size_t H = oneD ? 1 : fShapeX[2], W = fShapeX[fDim + 1];
      const size_t KH = oneD ? 1 : fShapeW[2], KW = fShapeW[fDim + 1];
      const size_t OH = oneD ? 1 : fShapeY[2], OW = fShapeY[fDim + 1];
      const size_t ph = oneD ? 0 : fAttrPads[0], pw = fAttrPads[oneD ? 0 : 1];
      const size_t sh = oneD ? 1 : fAttrStrides[0], sw = fAttrStrides[oneD ? 0 : 1];
      const size_t dh = oneD ? 1 : fAttrDilations[0], dw = fAttrDilations[oneD ? 0 : 1];
      std::stringstream out;
      out << "\n//----  operator ConvTranspose " << OpName << "\n";
      out << SP << "Check(sofie_hip_conv_transpose2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNW << ", "
          << (fNB.empty() ? std::string("nullptr") : "tensor_" + fNB) << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0]) << ", "
          << fShapeX[1] << ", " << H << ", " << W << ", " << fShapeY[1] << ", " << KH << ", " << KW << ", " << ph << ", " << pw
          << ", " << sh << ", " << sw << ", " << dh << ", " << dw << ", " << fAttrGroup << ", " << OH << ", " << OW << ", "
          << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << "), \"ConvTranspose " << OpName
          << "\");\n";
      return out.str();
   }

   // Host form, the reference's sequence for the transposed convolution (ROperator_ConvTranspose.icc:364-474 computes
   // it as a convolution of the zero-stuffed input with the flipped kernel; here the equivalent product-then-scatter):
   // per image and group one BLAS::sgemm_ multiplies the [H*W, C/g] input with the group's [C/g, OC/g*KH*KW] weights,
   // and every column of the result is added into the output at the positions its kernel cell reaches (stride,
   // dilation, begin pads); the bias and the ReLU follow.
   std::string GenerateHostSessionMembersCode(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeY.empty()) throw std::runtime_error("TMVA SOFIE ConvTranspose Op called to Generate without being initialized first");
      size_t in = 1, cells = 1;
      for (size_t i = 0; i < fDim; ++i) { in *= fShapeX[2 + i]; cells *= fShapeW[2 + i]; }
      return "std::vector<float> fVec_" + OpName + "_col = std::vector<float>(" + std::to_string(fShapeW[1] * cells * in) + ");\n";
   }
   std::string GenerateHost(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeW.empty() || (fNB != "" && fShapeB.empty()) || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Conv Op called to Generate without being initialized first");
      const bool oneD = fDim == 1;
      const size_t H = oneD ? 1 : fShapeX[2], W = fShapeX[fDim + 1];
      const size_t KH = oneD ? 1 : fShapeW[2], KW = fShapeW[fDim + 1];
      const size_t OH = oneD ? 1 : fShapeY[2], OW = fShapeY[fDim + 1];
      const size_t ph = oneD ? 0 : fAttrPads[0], pw = fAttrPads[oneD ? 0 : 1];
      const size_t sh = oneD ? 1 : fAttrStrides[0], sw = fAttrStrides[oneD ? 0 : 1];
      const size_t dh = oneD ? 1 : fAttrDilations[0], dw = fAttrDilations[oneD ? 0 : 1];
      const size_t C = fShapeX[1], OC = fShapeY[1], G = fAttrGroup, Cg = C / G, OCg = OC / G;
      std::stringstream out;
      out << "\n//----  operator ConvTranspose " << OpName << "\n";
      out << SP << "{\n";
      out << SP << SP << "char " << OpName << "_transA = 'N';\n";
      out << SP << SP << "char " << OpName << "_transB = 'T';\n";
      out << SP << SP << "int " << OpName << "_m = " << H * W << ";\n";
      out << SP << SP << "int " << OpName << "_n = " << OCg * KH * KW << ";\n";
      out << SP << SP << "int " << OpName << "_k = " << Cg << ";\n";
      out << SP << SP << "float " << OpName << "_alpha = 1.0;\n";
      out << SP << SP << "float " << OpName << "_beta = 0.0;\n";
      out << SP << SP << "float * " << OpName << "_col = fVec_" << OpName << "_col.data();\n";
      out << SP << SP << "std::fill_n(tensor_" << fNY << ", " << BatchCount(ConvertShapeToLength(fShapeY)) << ", 0.f);\n";
      out << SP << SP << "for (size_t n = 0; n < " << BatchCount(fShapeX[0]) << "; n++) {\n";
      out << SP << SP << SP << "for (size_t g = 0; g < " << G << "; g++) {\n";
      out << SP << SP << SP << SP << "BLAS::sgemm_(&" << OpName << "_transA, &" << OpName << "_transB, &" << OpName << "_m, &" << OpName
          << "_n, &" << OpName << "_k, &" << OpName << "_alpha, tensor_" << fNX << " + (n * " << C << " + g * " << Cg << ") * " << H * W << ", &"
          << OpName << "_m, tensor_" << fNW << " + g * " << Cg * OCg * KH * KW << ", &" << OpName << "_n, &" << OpName << "_beta, " << OpName
          << "_col, &" << OpName << "_m);\n";
      out << SP << SP << SP << SP << "Col2im(" << OpName << "_col, " << OCg << ", " << H << ", " << W << ", " << KH << ", " << KW << ", " << ph << ", "
          << pw << ", " << sh << ", " << sw << ", " << dh << ", " << dw << ", " << OH << ", " << OW << ", tensor_" << fNY << " + (n * " << OC
          << " + g * " << OCg << ") * " << OH * OW << ");\n";
      out << SP << SP << SP << "}\n";
      out << SP << SP << "}\n";
      if (fNB != "" || fActivation == EActivationType::RELU) {
         out << SP << SP << "for (size_t id = 0; id < " << BatchCount(ConvertShapeToLength(fShapeY)) << "; id++) {\n";
         out << SP << SP << SP << "float v = tensor_" << fNY << "[id]";
         if (fNB != "") out << " + tensor_" << fNB << "[(id / " << OH * OW << ") % " << OC << "]";
         out << ";\n";
         if (fActivation == EActivationType::RELU) out << SP << SP << SP << "v = v > 0 ? v : 0;\n";
         out << SP << SP << SP << "tensor_" << fNY << "[id] = v;\n";
         out << SP << SP << "}\n";
      }
      out << SP << "}\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
