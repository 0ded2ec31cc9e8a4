// Relu emitter; same interface as the reference's ROperator_Relu<T> (ROperator_Relu.hxx:17-66).
// Works on float tensors (kernel) and on int8 tensors (max with the zero-point is expressed by the
// producer's fused clamp, so a stand-alone int8 Relu is rejected).
#ifndef SOFIE_ROPERATOR_RELU
#define SOFIE_ROPERATOR_RELU

#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

template <typename T>
class ROperator_Relu final : public ROperator {
private:
   std::string fNX, fNY;
   std::vector<size_t> fShape;
   ETensorType fType = ETensorType::UNDEFINED;

public:
   ROperator_Relu() {}
   ROperator_Relu(std::string nameX, std::string nameY) : fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "Relu"; }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return input; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override { return input; }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE Relu Op Input Tensor " + fNX + " is not found in model");
      fShape = model.GetTensorShape(fNX);
      fType = model.GetTensorType(fNX);
      model.AddIntermediateTensor(fNY, fType, fShape);
      std::vector<size_t> chw;   // element-wise: the output keeps the input's memory order
      if (model.IsChannelsLast(fNX, &chw)) model.MarkChannelsLast(fNY, chw[0], chw[1], chw[2]);
   }
   std::string Generate(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShape.empty()) throw std::runtime_error("TMVA SOFIE Operator Relu called to Generate without being initialized first");
      if (fType != ETensorType::FLOAT)
         throw std::runtime_error("TMVA SOFIE Relu Op " + OpName + ": a Relu on a quantized tensor must follow the operator it can fuse with");
      std::stringstream out;
      out << "\n//------ RELU\n";
      out << SP << "Check(sofie_hip_relu_f32(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(ConvertShapeToLength(fShape))
          << "), \"Relu " << OpName << "\");\n";
      return out.str();
   }
   // what the loop of the reference's ROperator_Relu.hxx:54-66 computes, as one std::transform
   std::string GenerateHost(std::string OpName) override
   {
      OpName = "op_" + OpName;
      if (fShape.empty()) throw std::runtime_error("TMVA SOFIE Operator Relu called to Generate without being initialized first");
      if (fType != ETensorType::FLOAT) throw std::runtime_error("TMVA SOFIE Relu Op " + OpName + ": the host emission takes float tensors");
      std::stringstream out;
      out << "\n//------ RELU\n";
      const std::string count = BatchCount(ConvertShapeToLength(fShape));
      out << SP << "std::transform(tensor_" << fNX << ", tensor_" << fNX << " + " << count << ", tensor_" << fNY
          << ", [](float v) { return v > 0 ? v : 0.0f; });\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
