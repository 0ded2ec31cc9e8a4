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
      if (input[0].size() != 4)
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : tensors with dimension " + std::to_string(input[0].size()) +
                                  " are not yet supported");
      if (fPoolMode == GlobalAveragePool) {
         // a pooling whose kernel is the image (reference :216-228)
         fAttr.kernel_shape = {input[0][2], input[0][3]};
         fAttr.auto_pad = "NOTSET";
         fAttr.pads = {0, 0, 0, 0};
         fAttr.strides = {1, 1};
      }
      if (fAttr.kernel_shape.empty()) fAttr.kernel_shape = {input[0][2], input[0][3]};
      if (fAttr.auto_pad != "NOTSET")
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : auto_pad is not supported by the device emission");
      if (fAttr.ceil_mode != 0)
         throw std::runtime_error("TMVA SOFIE" + Name() + "Op : ceil_mode is not supported by the device emission");
      if (fAttr.pads.empty()) fAttr.pads = {0, 0, 0, 0};
      fAttr.pads.resize(4, 0);
      if (fAttr.strides.empty()) fAttr.strides = {1, 1};
      for (auto d : fAttr.dilations)
         if (d != 1) throw std::runtime_error("TMVA SOFIE" + Name() + "Op : dilations are not supported by the device emission");
      const size_t oh = (input[0][2] + fAttr.pads[0] + fAttr.pads[2] - fAttr.kernel_shape[0]) / fAttr.strides[0] + 1;
      const size_t ow = (input[0][3] + fAttr.pads[1] + fAttr.pads[3] - fAttr.kernel_shape[1]) / fAttr.strides[1] + 1;
      return {{input[0][0], input[0][1], oh, ow}};
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
      fChannelsLast = model.IsChannelsLast(fNX);
      if (fChannelsLast) model.MarkChannelsLast(fNY, fShapeY[1], fShapeY[2], fShapeY[3]);
   }
   std::string Generate(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShapeX.empty() || fShapeY.empty())
         throw std::runtime_error("TMVA SOFIE Pool Op called to Generate without being initialized first");
      std::stringstream out;
      out << "\n//----  operator " << Name() << "  " << OpName << "\n";
      const auto &a = fAttr;
      if (fPoolMode != MaxPool) {
         // a window that lies in the padding entirely has no cell to average
         if (!a.count_include_pad)
            for (size_t i = 0; i < 4; ++i)
               if (a.pads[i] >= a.kernel_shape[i % 2])
                  throw std::runtime_error("TMVA SOFIE" + Name() + "Op : a pad as large as the kernel leaves windows without a cell of the image");
         out << SP << "Check(sofie_hip_avgpool2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0] * fShapeX[1])
             << ", " << fShapeX[2] << ", " << fShapeX[3] << ", " << a.kernel_shape[0] << ", " << a.kernel_shape[1] << ", " << a.pads[0]
             << ", " << a.pads[1] << ", " << a.pads[2] << ", " << a.pads[3] << ", " << a.strides[0] << ", " << a.strides[1] << ", "
             << (a.count_include_pad ? 1 : 0) << "), \"" << Name() << " " << OpName << "\");\n";
         return out.str();
      }
      if (fType == ETensorType::FLOAT)
         out << SP << "Check(sofie_hip_maxpool2d_f32(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(fShapeX[0] * fShapeX[1])
             << ", " << fShapeX[2] << ", " << fShapeX[3];
      else
         out << SP << "Check(sofie_hip_maxpool2d_s8(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << (fChannelsLast ? "SOFIE_LAYOUT_NHWC" : "SOFIE_LAYOUT_NCHW") << ", "
             << BatchCount(fShapeX[0]) << ", " << fShapeX[1] << ", " << fShapeX[2] << ", " << fShapeX[3];
      out << ", " << a.kernel_shape[0] << ", " << a.kernel_shape[1] << ", " << a.pads[0] << ", " << a.pads[1] << ", " << a.pads[2]
          << ", " << a.pads[3] << ", " << a.strides[0] << ", " << a.strides[1] << "), \"" << Name() << " " << OpName << "\");\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
