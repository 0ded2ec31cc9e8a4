// Pooling emitter; interface of the reference's ROperator_Pool<T> (ROperator_Pool.hxx:17-90): a mode,
// an attribute struct, input and output names. The device emission covers 2-D MaxPool (float NCHW and
// int8 in either layout), 2-D AveragePool and GlobalAveragePool (float NCHW; the latter is the average over the
// whole image, as the reference turns it into at Initialize, :216-228), with the reference's output-size rule
// (floor division, default pads 0, :92-199).
#ifndef SOFIE_ROPERATOR_POOL
#define SOFIE_ROPERATOR_POOL

#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

struct RAttributes_Pool {
   std::string auto_pad = "NOTSET";
   int ceil_mode = 0;
   int count_include_pad = 0;
   int storage_order = 0;
   std::vector<size_t> dilations;
   std::vector<size_t> kernel_shape;
   std::vector<size_t> pads;
   std::vector<size_t> strides;
};

enum PoolOpMode { InvalidPool, MaxPool, AveragePool, GlobalAveragePool };

template <typename T>
class ROperator_Pool final : public ROperator {
private:
   PoolOpMode fPoolMode;
   RAttributes_Pool fAttr;
   std::string fNX, fNY;
   std::vector<size_t> fShapeX, fShapeY;
   ETensorType fType = ETensorType::UNDEFINED;
   bool fChannelsLast = false;   // int8 input stored [N,H,W,C]

public:
   ROperator_Pool() {}
   ROperator_Pool(PoolOpMode mode, RAttributes_Pool attr, std::string nameX, std::string nameY)
      : fPoolMode(mode), fAttr(attr), fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "Pool"; }
   // what a producer needs to know to absorb this pooling (valid after Initialize)
   bool IsPlainMaxPool() const
   {
      if (fPoolMode != MaxPool || fAttr.ceil_mode != 0) return false;
      for (auto p : fAttr.pads)
         if (p != 0) return false;
      return fAttr.kernel_shape.size() == 2 && fAttr.strides.size() == 2;
   }
   const std::vector<size_t> &KernelShape() const { return fAttr.kernel_shape; }
   const std::vector<size_t> &Strides() const { return fAttr.strides; }
   const std::vector<size_t> &OutputShape() const { return fShapeY; }
   ETensorType TensorType() const { return fType; }
   std::string Name()
   {
      return fPoolMode == MaxPool ? "MaxPool" : fPoolMode == AveragePool ? "AveragePool"
             : fPoolMode == GlobalAveragePool ? "GlobalAveragePool" : "Invalid";
   }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return input; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      if (input.size() != 1) throw std::runtime_error("TMVA SOFIE" + Name() + "Op Shape inference need 1 input tensor");
      // one, two or three spatial axes behind [N, C] (reference :102-105)
      if (input[0].size() < 3 || input[0].size() > 5)
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : tensors with dimension " + std::to_string(input[0].size()) +
                                  " are not yet supported");
      const size_t dims = input[0].size() - 2;
      const std::vector<size_t> spatial(input[0].begin() + 2, input[0].end());
      if (fPoolMode == GlobalAveragePool) {
         // a pooling whose kernel is the image (reference :216-228)
         fAttr.kernel_shape = spatial;
         fAttr.auto_pad = "NOTSET";
         fAttr.pads.assign(2 * dims, 0);
         fAttr.strides.assign(dims, 1);
      }
      if (fAttr.kernel_shape.empty()) fAttr.kernel_shape = spatial;
      if (fAttr.kernel_shape.size() != dims)
         throw std::runtime_error("TMVA SOFIE Pool Op Shape inference - invalid inputs ");
      if (fAttr.auto_pad != "NOTSET")
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : auto_pad is not supported by the device emission");
      if (fAttr.ceil_mode != 0)
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : ceil_mode is not supported by the device emission");
      // pads in ONNX order: the begin pads of the axes, then their end pads
      if (fAttr.pads.empty()) fAttr.pads.assign(2 * dims, 0);
      if (fAttr.pads.size() != 2 * dims)
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : " + std::to_string(fAttr.pads.size()) + " pads for " +
                                  std::to_string(dims) + " spatial axes");
      if (fAttr.strides.empty()) fAttr.strides.assign(dims, 1);
      if (fAttr.strides.size() != dims)
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : " + std::to_string(fAttr.strides.size()) + " strides for " +
                                  std::to_string(dims) + " spatial axes");
      for (auto d : fAttr.dilations)
         if (d != 1) throw std::runtime_error("TMVA SOFIE" + Name() + "Op : dilations are not supported by the device emission");
      std::vector<size_t> out = {input[0][0], input[0][1]};
      for (size_t i = 0; i < dims; ++i) {
         if (spatial[i] + fAttr.pads[i] + fAttr.pads[dims + i] < fAttr.kernel_shape[i] || fAttr.strides[i] == 0)
            throw std::runtime_error("TMVA SOFIE" + Name() + "Op : kernel larger than the padded input");
         out.push_back((spatial[i] + fAttr.pads[i] + fAttr.pads[dims + i] - fAttr.kernel_shape[i]) / fAttr.strides[i] + 1);
      }
      return {out};
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE Pool op Input Tensor " + fNX + " is not found in model");
      if (fPoolMode != MaxPool && fPoolMode != AveragePool && fPoolMode != GlobalAveragePool)
         throw std::runtime_error("TMVA SOFIE Pool op " + Name() + " is not supported by the device emission");
      fShapeX = model.GetTensorShape(fNX);
      fType = model.GetTensorType(fNX);
      if (fType != ETensorType::FLOAT && fType != ETensorType::INT8)
         throw std::runtime_error("TMVA SOFIE Encountered unsupported type parsing a Pool operator");
      if (fPoolMode != MaxPool && fType != ETensorType::FLOAT)
         throw std::runtime_error("TMVA SOFIE Pool op " + Name() + " on a quantized tensor is not supported by the device emission");
      fShapeY = ShapeInference({fShapeX})[0];
      model.AddIntermediateTensor(fNY, fType, fShapeY);
      fChannelsLast = fShapeX.size() == 4 && model.IsChannelsLast(fNX);
      if (fChannelsLast) model.MarkChannelsLast(fNY, fShapeY[1], fShapeY[2], fShapeY[3]);
      if (fShapeX.size() == 5 && fType != ETensorType::FLOAT)
         throw std::runtime_error("TMVA SOFIE Pool op " + Name() + " over three spatial axes on a quantized tensor is not supported by the device emission");
   }
   std::string Generate(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Pool Op called to Generate without being initialized first");
      std::stringstream out;
      out << "\n//----  operator " << Name() << "  " << OpName << "\n";
      const size_t dims = fShapeX.size() - 2;
      // a window that lies in the padding entirely has no cell to average
      if (fPoolMode != MaxPool && !fAttr.count_include_pad)
         for (size_t i = 0; i < 2 * dims; ++i)
            if (fAttr.pads[i] >= fAttr.kernel_shape[i % dims])
               throw std::runtime_error("TMVA SOFIE" + Name() + "Op : a pad as large as the kernel leaves windows without a cell of the image");
      if (dims == 3) {
         // three spatial axes (reference :417-470): geometry as arrays, pads in ONNX order
         auto list = [](const std::vector<size_t> &v) {
            std::string t = "{";
            for (size_t i = 0; i < v.size(); ++i) t += (i ? ", " : "") + std::to_string(v[i]);
            return t + "}";
         };
         out << SP << "{\n";
         out << SP << SP << "const int dims[3] = " << list({fShapeX[2], fShapeX[3], fShapeX[4]}) << ", kernel[3] = " << list(fAttr.kernel_shape)
             << ", pads[6] = " << list(fAttr.pads) << ", strides[3] = " << list(fAttr.strides) << ";\n";
         out << SP << SP << "Check(sofie_hip_" << (fPoolMode == MaxPool ? "maxpool3d_f32" : "avgpool3d_f32") << "(fCtx, tensor_" << fNX << ", tensor_"
             << fNY << ", " << BatchCount(fShapeX[0] * fShapeX[1]) << ", dims, kernel, pads, strides";
         if (fPoolMode != MaxPool) out << ", " << (fAttr.count_include_pad ? 1 : 0);
         out << "), \"" << Name() << " " << OpName << "\");\n";
         out << SP << "}\n";
         return out.str();
      }
      // one spatial axis (reference :329-370) is the two-axis call on [N*C, 1, W] with a 1 x k window
      struct Geometry2d {
         size_t H, W, kh, kw, pt, pl, pb, pr, sh, sw;
      } a;
      if (dims == 1)
         a = {1, fShapeX[2], 1, fAttr.kernel_shape[0], 0, fAttr.pads[0], 0, fAttr.pads[1], 1, fAttr.strides[0]};
      else
         a = {fShapeX[2], fShapeX[3], fAttr.kernel_shape[0], fAttr.kernel_shape[1], fAttr.pads[0], fAttr.pads[1], fAttr.pads[2],
              fAttr.pads[3], fAttr.strides[0], fAttr.strides[1]};
      if (fPoolMode != MaxPool) {
         out << SP << "Check(sofie_hip_avgpool2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0] * fShapeX[1])
             << ", " << a.H << ", " << a.W << ", " << a.kh << ", " << a.kw << ", " << a.pt << ", " << a.pl << ", " << a.pb << ", " << a.pr
             << ", " << a.sh << ", " << a.sw << ", " << (fAttr.count_include_pad ? 1 : 0) << "), \"" << Name() << " " << OpName << "\");\n";
         return out.str();
      }
      if (fType == ETensorType::FLOAT)
         out << SP << "Check(sofie_hip_maxpool2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0] * fShapeX[1])
             << ", " << a.H << ", " << a.W;
      else
         out << SP << "Check(sofie_hip_maxpool2d_s8(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << (fChannelsLast ? "SOFIE_LAYOUT_NHWC" : "SOFIE_LAYOUT_NCHW") << ", "
             << BatchCount(fShapeX[0]) << ", " << fShapeX[1] << ", " << a.H << ", " << a.W;
      out << ", " << a.kh << ", " << a.kw << ", " << a.pt << ", " << a.pl << ", " << a.pb << ", " << a.pr << ", " << a.sh << ", " << a.sw
          << "), \"" << Name() << " " << OpName << "\");\n";
      return out.str();
   }

   // Host form: the loops of the reference's pooling (ROperator_Pool.hxx:266-476) over one, two or three spatial
   // axes, as one helper of the generated file (Pool3d; missing leading axes have extent 1). A window takes the cells
   // that lie inside the image; the average divides by their number, or by the kernel's size with count_include_pad.
   std::string GenerateHost(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Pool Op called to Generate without being initialized first");
      const size_t dims = fShapeX.size() - 2;
      if (fType != ETensorType::FLOAT) {
         // int8 max pooling over two axes, on [N,C,H,W] or on the channels-last tensor of the quantized operators
         if (fPoolMode != MaxPool || dims != 2) throw std::runtime_error("TMVA SOFIE Pool Op " + OpName + ": no host emission for this int8 pooling");
         std::stringstream q;
         q << "\n//----  operator MaxPool (int8)  " << OpName << "\n";
         q << SP << "MaxPoolInt8(tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0]) << ", " << fShapeX[1] << ", " << fShapeX[2]
           << ", " << fShapeX[3] << ", " << fAttr.kernel_shape[0] << ", " << fAttr.kernel_shape[1] << ", " << fAttr.pads[0] << ", " << fAttr.pads[1]
           << ", " << fAttr.strides[0] << ", " << fAttr.strides[1] << ", " << fShapeY[2] << ", " << fShapeY[3] << ", "
           << (fChannelsLast ? "true" : "false") << ");\n";
         return q.str();
      }
      if (fPoolMode != MaxPool && !fAttr.count_include_pad)
         for (size_t i = 0; i < 2 * dims; ++i)
            if (fAttr.pads[i] >= fAttr.kernel_shape[i % dims])
               throw std::runtime_error("TMVA SOFIE" + Name() + "Op : a pad as large as the kernel leaves windows without a cell of the image");
      // three axes, the given ones last
      size_t in[3] = {1, 1, 1}, o[3] = {1, 1, 1}, k[3] = {1, 1, 1}, pb[3] = {0, 0, 0}, st[3] = {1, 1, 1};
      for (size_t i = 0; i < dims; ++i) {
         const size_t a = 3 - dims + i;
         in[a] = fShapeX[2 + i]; o[a] = fShapeY[2 + i]; k[a] = fAttr.kernel_shape[i]; pb[a] = fAttr.pads[i]; st[a] = fAttr.strides[i];
      }
      auto list = [](const size_t (&v)[3]) { return "{" + std::to_string(v[0]) + ", " + std::to_string(v[1]) + ", " + std::to_string(v[2]) + "}"; };
      std::stringstream out;
      out << "\n//----  operator " << Name() << "  " << OpName << "\n";
      out << SP << "{\n";
      out << SP << SP << "const int " << OpName << "_in[3] = " << list(in) << ", " << OpName << "_out[3] = " << list(o) << ", " << OpName
          << "_kernel[3] = " << list(k) << ", " << OpName << "_pads[3] = " << list(pb) << ", " << OpName << "_strides[3] = " << list(st) << ";\n";
      out << SP << SP << "Pool3d(" << (fPoolMode == MaxPool ? "true" : "false") << ", " << (fAttr.count_include_pad ? "true" : "false") << ", tensor_"
          << fNX << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0] * fShapeX[1]) << ", " << OpName << "_in, " << OpName << "_out, " << OpName
          << "_kernel, " << OpName << "_pads, " << OpName << "_strides);\n";
      out << SP << "}\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
