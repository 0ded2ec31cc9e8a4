// Conv emitter (1-D, 2-D and 3-D). Constructor, attribute defaults, output-shape rule and error messages follow the
// reference's ROperator_Conv<T> (src/SOFIE_core/inc/SOFIE/ROperator_Conv.hxx:52-87,95-201,203-282):
//   - auto_pad NOTSET with no pads attribute means 1 on every side (:136-139, not ONNX's 0);
//   - group == 0 means C / C_w (:110-112).
// Two rules of the reference are NOT followed, because they make its own generated code inconsistent:
//   - SAME_UPPER / SAME_LOWER: the reference starts from k/2 on both sides and adds one at the begin / end for odd
//     kernels (:140-158), i.e. a total of k for a 3x3 kernel; the output shape it declares then has one row and column
//     more than the averaged pad of its Im2col call writes. Here the pads are ONNX's: the total that makes the output
//     ceil(in / stride), the odd unit at the end (SAME_UPPER) or at the begin (SAME_LOWER);
//   - begin/end pads that differ: the reference averages them with a warning (:387-401) while the declared output
//     shape uses their sum. Here the kernel library takes all four pads and the result is ONNX's.
// Emitted code: one sofie_hip_conv2d_f32 call over the whole batch (implicit GEMM, bias and
// optional ReLU fused) instead of the per-image weight re-layout + Im2col + sgemm_ + saxpy_. A 1-D operator
// [N,C,W] runs as the 2-D one on [N,C,1,W] (the reference does the same inside Im2col, :424-427); a 3-D one is
// one sofie_hip_conv3d_f32 call where the reference emits Im2col_3d + sgemm_ (:432-451).
// Dilation: the reference hands Im2col the dilated kernel extent together with the dilation (:118-122,:418-444),
// which counts the dilation twice; here the kernel size is the weight tensor's and the dilation is applied once,
// as ONNX defines it.
#ifndef SOFIE_SOFIE_ROPERATOR_CONV
#define SOFIE_SOFIE_ROPERATOR_CONV

#include <cstdlib>
#include <iostream>
#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

// Attribute handling shared by Conv and QLinearConv, for 1, 2 or 3 spatial dimensions (the reference's fDim,
// ROperator_Conv.hxx:95-201). After Resolve every attribute vector has `dim` entries (pads 2*dim: begins, then ends).
struct ConvGeometry {
   std::string autopad;
   std::vector<size_t> dilations, kernel, pads, strides;
   size_t group = 0;
   size_t dim = 2;
   // fills defaults, returns the output shape [N, OC, o1, ..] for input [N,C,i1,..] and weights [OC,C/g,k1,..]
   std::vector<size_t> Resolve(const std::vector<size_t> &x, const std::vector<size_t> &w)
   {
      if (x.size() < 3 || x.size() > 5 || w.size() != x.size())
         throw std::runtime_error("TMVA SOFIE Conv Op Shape inference - invalid inputs ");
      dim = x.size() - 2;
      if (group == 0) group = x[1] / w[1];
      if (!kernel.empty() && kernel.size() != dim)
         throw std::runtime_error("TMVA SOFIE Conv Op: kernel_shape does not match the number of spatial dimensions");
      std::vector<size_t> k(dim), extent(dim);
      for (size_t i = 0; i < dim; ++i) k[i] = kernel.empty() ? w[i + 2] : kernel[i];
      kernel = k;
      if (dilations.empty()) dilations.assign(dim, 1);
      dilations.resize(dim, 1);
      // dilated extent of the kernel
      for (size_t i = 0; i < dim; ++i) extent[i] = k[i] + (dilations[i] - 1) * (k[i] - 1);
      if (autopad == "NOTSET" || autopad == "") {
         if (pads.empty()) pads.assign(2 * dim, 1);
      } else if (autopad == "SAME_UPPER" || autopad == "SAME_LOWER") {
         if (strides.empty()) strides.assign(dim, 1);
         strides.resize(dim, 1);
         pads.assign(2 * dim, 0);
         for (size_t i = 0; i < dim; ++i) {
            const size_t in = x[i + 2], st = strides[i];
            const size_t covered = ((in + st - 1) / st - 1) * st + extent[i];   // reach of the last of ceil(in/st) windows
            const size_t total = covered > in ? covered - in : 0;
            const size_t small = total / 2, large = total - small;
            pads[i] = autopad == "SAME_UPPER" ? small : large;
            pads[dim + i] = autopad == "SAME_UPPER" ? large : small;
         }
      } else if (autopad == "VALID") {
         pads.assign(2 * dim, 0);
      } else {
         throw std::runtime_error("TMVA SOFIE Conv Op invalid fAutopad");
      }
      pads.resize(2 * dim, 0);
      if (strides.empty()) strides.assign(dim, 1);
      strides.resize(dim, 1);
      std::vector<size_t> out = {x[0], w[0]};
      for (size_t i = 0; i < dim; ++i) out.push_back((x[i + 2] + pads[i] + pads[dim + i] - extent[i]) / strides[i] + 1);
      return out;
   }
   // the four pads of a 2-D operator in ONNX order (top, left, bottom, right)
   void Pads2D(size_t &pt, size_t &pl, size_t &pb, size_t &pr) const
   {
      if (dim != 2) throw std::runtime_error("TMVA SOFIE Conv Op: a 2-D convolution is expected here");
      pt = pads[0]; pl = pads[1]; pb = pads[2]; pr = pads[3];
   }
   // 3-D operators: the kernel takes one pad per axis
   std::vector<size_t> EqualPads() const
   {
      for (size_t i = 0; i < dim; ++i)
         if (pads[i] != pads[dim + i])
            throw std::runtime_error("TMVA SOFIE Conv Op: begin and end pads that differ are not supported for 3-D convolutions");
      return std::vector<size_t>(pads.begin(), pads.begin() + dim);
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
      if (fShapeX.size() < 3 || fShapeX.size() > 5)
         throw std::runtime_error("TMVA SOFIE Conv Op input data tensor" + fNX + " is not of 3,4 or 5 dimensions");
      if (!model.CheckIfTensorAlreadyExist(fNW))
         throw std::runtime_error("TMVA SOFIE Conv op Input weight Tensor " + fNW + " is not found in model");
      fShapeW = model.GetTensorShape(fNW);
      if (fShapeW.size() < 3 || fShapeW.size() > 5 || fShapeW.size() != fShapeX.size())
         throw std::runtime_error("TMVA SOFIE Conv Op input weight tensor" + fNW + " is not of 3,4 or 5 dimensions");
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
      const size_t dim = fGeom.dim;
      const std::string bias = fNB.empty() ? std::string("nullptr") : "tensor_" + fNB;
      const std::string act = fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE";
      std::stringstream out;
      out << "\n//----  operator Conv " << OpName << "\n";
      if (dim == 3) {
         out << SP << "Check(sofie_hip_conv3d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNW << ", " << bias << ", tensor_" << fNY;
         out << ", " << BatchCount(fShapeX[0]);
         for (size_t i = 1; i < 5; ++i) out << ", " << fShapeX[i];
         out << ", " << fShapeW[0];
         for (size_t i = 0; i < 3; ++i) out << ", " << fShapeW[2 + i];
         const std::vector<size_t> p = fGeom.EqualPads();
         for (size_t i = 0; i < 3; ++i) out << ", " << p[i];
         for (size_t i = 0; i < 3; ++i) out << ", " << fGeom.strides[i];
         for (size_t i = 0; i < 3; ++i) out << ", " << fGeom.dilations[i];
         out << ", " << fGeom.group << ", " << act << "), \"Conv " << OpName << "\");\n";
         return out.str();
      }
      // one spatial dimension: a height of one, no padding and a unit stride along it
      const bool oneD = dim == 1;
      const size_t H = oneD ? 1 : fShapeX[2], W = fShapeX[dim + 1];
      const size_t KH = oneD ? 1 : fShapeW[2], KW = fShapeW[dim + 1];
      const std::vector<size_t> &p = fGeom.pads;   // begins, then ends
      const size_t pt = oneD ? 0 : p[0], pl = p[dim - 1], pb = oneD ? 0 : p[dim], pr = p[2 * dim - 1];
      const size_t sh = oneD ? 1 : fGeom.strides[0], sw = fGeom.strides[dim - 1];
      const size_t dh = oneD ? 1 : fGeom.dilations[0], dw = fGeom.dilations[dim - 1];
      out << SP << "Check(sofie_hip_conv2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNW << ", " << bias << ", tensor_" << fNY << ", "
          << BatchCount(fShapeX[0]) << ", " << fShapeX[1] << ", " << H << ", " << W << ", " << fShapeW[0] << ", " << KH << ", " << KW << ", " << pt
          << ", " << pl << ", " << pb << ", " << pr << ", " << sh << ", " << sw << ", " << dh << ", " << dw << ", " << fGeom.group << ", " << act << "), \"Conv "
          << OpName << "\");\n";
      return out.str();
   }

   // Host form, the reference's sequence (ROperator_Conv.hxx:302-522): per image (and group) the patches are laid out
   // as a column-major [OH*OW, C/g*KH*KW] matrix (Im2col), one BLAS::sgemm_ multiplies it with the group's filters
   // (the [OC/g, C/g*KH*KW] rows of the weight tensor are that matrix's column-major transpose already), and the
   // bias, broadcast to [OC,OH,OW] once in the constructor, is added with BLAS::saxpy_; then the ReLU loop. The
   // geometry is this emitter's (ONNX pads and dilations, see the head of the file), through one Im2col for one, two
   // or three spatial axes (the reference's Im2col and Im2col_3d).
   std::string GenerateHostSessionMembersCode(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeY.empty()) throw std::runtime_error("TMVA SOFIE Conv Op called to Generate without being initialized first");
      size_t spatialOut = 1, kernelCells = 1;
      for (size_t i = 0; i < fGeom.dim; ++i) { spatialOut *= fShapeY[2 + i]; kernelCells *= fShapeW[2 + i]; }
      std::stringstream out;
      out << "std::vector<float> fVec_" << OpName << "_xcol = std::vector<float>(" << fShapeW[1] * kernelCells * spatialOut << ");\n";
      if (fNB != "") out << "std::vector<float> fVec_" << OpName << "_bias = std::vector<float>(" << fShapeY[1] * spatialOut << ");\n";
      return out.str();
   }
   std::string GenerateHostInitCode(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fNB == "") return "";
      size_t spatialOut = 1;
      for (size_t i = 0; i < fGeom.dim; ++i) spatialOut *= fShapeY[2 + i];
      std::stringstream out;
      out << SP << "for (size_t oc = 0; oc < " << fShapeY[1] << "; ++oc) std::fill_n(fVec_" << OpName << "_bias.data() + oc * " << spatialOut
          << ", " << spatialOut << ", tensor_" << fNB << "[oc]);\n";
      return out.str();
   }
   std::string GenerateHost(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeW.empty() || (fNB != "" && fShapeB.empty()) || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Conv Op called to Generate without being initialized first");
      const size_t dim = fGeom.dim;
      // three spatial axes, the given ones last (missing leading axes have extent 1, no padding, unit stride)
      size_t in[3] = {1, 1, 1}, ker[3] = {1, 1, 1}, o[3] = {1, 1, 1}, pad[3] = {0, 0, 0}, st[3] = {1, 1, 1}, dil[3] = {1, 1, 1};
      for (size_t i = 0; i < dim; ++i) {
         const size_t a = 3 - dim + i;
         in[a] = fShapeX[2 + i]; ker[a] = fShapeW[2 + i]; o[a] = fShapeY[2 + i]; pad[a] = fGeom.pads[i]; st[a] = fGeom.strides[i];
         dil[a] = fGeom.dilations[i];
      }
      const size_t inSize = in[0] * in[1] * in[2], kerSize = ker[0] * ker[1] * ker[2], outSize = o[0] * o[1] * o[2];
      const size_t C = fShapeX[1], OC = fShapeW[0], G = fGeom.group, Cg = fShapeW[1], OCg = OC / G;
      auto list = [](const size_t (&v)[3]) { return "{" + std::to_string(v[0]) + ", " + std::to_string(v[1]) + ", " + std::to_string(v[2]) + "}"; };
      std::stringstream out;
      out << "\n//----  operator Conv " << OpName << "\n";
      out << SP << "{\n";
      out << SP << SP << "char " << OpName << "_transA = 'N';\n";
      out << SP << SP << "char " << OpName << "_transB = 'N';\n";
      out << SP << SP << "int " << OpName << "_m = " << outSize << ";\n";
      out << SP << SP << "int " << OpName << "_n = " << OCg << ";\n";
      out << SP << SP << "int " << OpName << "_k = " << Cg * kerSize << ";\n";
      out << SP << SP << "float " << OpName << "_alpha = 1.0;\n";
      out << SP << SP << "float " << OpName << "_beta = 0.0;\n";
      out << SP << SP << "float * " << OpName << "_xcol = fVec_" << OpName << "_xcol.data();\n";
      out << SP << SP << "const int " << OpName << "_in[3] = " << list(in) << ", " << OpName << "_kernel[3] = " << list(ker) << ", " << OpName
          << "_pads[3] = " << list(pad) << ", " << OpName << "_strides[3] = " << list(st) << ", " << OpName << "_dilations[3] = " << list(dil)
          << ", " << OpName << "_out[3] = " << list(o) << ";\n";
      out << SP << SP << "for (size_t n = 0; n < " << BatchCount(fShapeX[0]) << "; n++) {\n";
      out << SP << SP << SP << "for (size_t g = 0; g < " << G << "; g++) {\n";
      out << SP << SP << SP << SP << "Im2col(tensor_" << fNX << " + (n * " << C << " + g * " << Cg << ") * " << inSize << ", " << Cg << ", " << OpName
          << "_in, " << OpName << "_kernel, " << OpName << "_pads, " << OpName << "_strides, " << OpName << "_dilations, " << OpName << "_out, "
          << OpName << "_xcol);\n";
      out << SP << SP << SP << SP << "BLAS::sgemm_(&" << OpName << "_transA, &" << OpName << "_transB, &" << OpName << "_m, &" << OpName
          << "_n, &" << OpName << "_k, &" << OpName << "_alpha, " << OpName << "_xcol, &" << OpName << "_m, tensor_" << fNW << " + g * "
          << OCg * Cg * kerSize << ", &" << OpName << "_k, &" << OpName << "_beta, tensor_" << fNY << " + (n * " << OC << " + g * " << OCg
          << ") * " << outSize << ", &" << OpName << "_m);\n";
      out << SP << SP << SP << "}\n";
      if (fNB != "") {
         out << SP << SP << SP << "int " << OpName << "_size = " << OC * outSize << ";\n";
         out << SP << SP << SP << "float " << OpName << "_gamma = 1.0;\n";
         out << SP << SP << SP << "int " << OpName << "_incx = 1;\n";
         out << SP << SP << SP << "int " << OpName << "_incy = 1;\n";
         out << SP << SP << SP << "BLAS::saxpy_(&" << OpName << "_size, &" << OpName << "_gamma, fVec_" << OpName << "_bias.data(), &" << OpName
             << "_incx, tensor_" << fNY << " + n * " << OC * outSize << ", &" << OpName << "_incy);\n";
      }
      out << SP << SP << "}\n";
      if (fActivation == EActivationType::RELU) {
         out << SP << SP << "for (size_t id = 0; id < " << BatchCount(ConvertShapeToLength(fShapeY)) << "; id++)\n";
         out << SP << SP << SP << "tensor_" << fNY << "[id] = ((tensor_" << fNY << "[id] > 0 )? tensor_" << fNY << "[id] : 0);\n";
      }
      out << SP << "}\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
