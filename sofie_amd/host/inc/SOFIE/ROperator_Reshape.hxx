// Reshape-family emitter; interface of the reference's ROperator_Reshape (ROperator_Reshape.hxx:17-80):
// (mode, attribute value, data name, shape name, output name). The device emission covers Flatten and
// a Reshape whose target shape is an initializer; both are views of the input buffer (the reference
// emits std::copy, :243-244).
#ifndef SOFIE_ROPERATOR_RESHAPE
#define SOFIE_ROPERATOR_RESHAPE

#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

enum ReshapeOpMode { Reshape, Flatten, Squeeze, Unsqueeze };

class ROperator_Reshape final : public ROperator {
private:
   ReshapeOpMode fOpMode = Reshape;
   int fAttrAxis = 1;   // Flatten axis (allowzero for Reshape, unused)
   std::string fNData, fNShape, fNOutput;
   std::vector<size_t> fShapeInput, fShapeOutput;

public:
   ROperator_Reshape() {}
   ROperator_Reshape(ReshapeOpMode opMode, int attr_value, std::string nameData, std::string nameShape, std::string nameOutput)
      : fOpMode(opMode), fAttrAxis(attr_value), fNData(UTILITY::Clean_name(nameData)), fNShape(UTILITY::Clean_name(nameShape)),
        fNOutput(UTILITY::Clean_name(nameOutput))
   {
      fInputTensorNames = {fNData};
      fOutputTensorNames = {fNOutput};
   }
   std::string Kind() const override { return "Reshape"; }
   std::string ViewOf() const override { return fNData; }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return {input[0]}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      const std::vector<size_t> &in = input[0];
      if (fOpMode == Flatten) {
         // [d0*..*d(axis-1), d(axis)*..*dn], negative axis counts from the end (reference :112-118)
         int axis = fAttrAxis < 0 ? fAttrAxis + (int)in.size() : fAttrAxis;
         size_t a = 1, b = 1;
         for (int i = 0; i < (int)in.size(); ++i) (i < axis ? a : b) *= in[i];
         return {{a, b}};
      }
      if (fOpMode == Reshape && input.size() == 2) {
         std::vector<size_t> out = input[1];
         size_t known = 1;
         int wild = -1;
         for (size_t i = 0; i < out.size(); ++i) {
            if (out[i] == (size_t)-1) wild = (int)i;
            else {
               if (out[i] == 0 && i < in.size()) out[i] = in[i];
               known *= out[i];
            }
         }
         if (wild >= 0) out[wild] = ConvertShapeToLength(in) / known;
         if (ConvertShapeToLength(out) != ConvertShapeToLength(in))
            throw std::runtime_error("TMVA Reshape Op : Invalid  shapes : " + ConvertShapeToString(in) + ConvertShapeToString(out));
         return {out};
      }
      throw std::runtime_error("TMVA SOFIE Reshape Op: mode not supported by the device emission");
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNData))
         throw std::runtime_error("TMVA Reshape Op Input Tensor " + fNData + "  is not found in model");
      fShapeInput = model.GetTensorShape(fNData);
      if (fOpMode == Flatten) {
         fShapeOutput = ShapeInference({fShapeInput})[0];
      } else {
         if (fNShape.empty() || !model.IsInitializedTensor(fNShape))
            throw std::runtime_error("TMVA Reshape Op Shape Tensor " + fNShape + " is not found in model");
         auto data = static_cast<int64_t *>(model.GetInitializedTensorData(fNShape).get());
         std::vector<size_t> target(data, data + ConvertShapeToLength(model.GetTensorShape(fNShape)));
         fShapeOutput = ShapeInference({fShapeInput, target})[0];
         model.SetNotWritableInitializedTensor(fNShape);
      }
      model.AddIntermediateTensor(fNOutput, model.GetTensorType(fNData), fShapeOutput);
      std::vector<size_t> chw;
      if (model.IsChannelsLast(fNData, &chw) && chw[0] > 1 && chw[1] * chw[2] > 1) {
         // the bytes stay in (h,w,c) order: only a flatten to [N, C*H*W] can be handed on, with the order recorded
         if (fShapeOutput.size() == 2 && fShapeOutput[0] == fShapeInput[0] && fShapeOutput[1] == chw[0] * chw[1] * chw[2])
            model.MarkChannelsLast(fNOutput, chw[0], chw[1], chw[2]);
         else
            throw std::runtime_error("TMVA Reshape Op: tensor " + fNData + " is stored channels-last and can only be flattened to [N, C*H*W]");
      }
   }
   std::string Generate(std::string OpName) override
   {
      if (fShapeInput.empty()) throw std::runtime_error("TMVA SOFIE Reshape Op called to Generate without being initialized first");
      // a view when the input lives in the arena; a graph input or a weight has to be copied
      return "\n//------ " + std::string(fOpMode == Flatten ? "FLATTEN" : "RESHAPE") + " op_" + OpName + " (view of tensor_" + fNData +
             ")\n" + SP + "if (static_cast<const void*>(tensor_" + fNOutput + ") != static_cast<const void*>(tensor_" + fNData +
             ")) Check(sofie_hip_copy(fCtx, tensor_" + fNOutput + ", tensor_" + fNData + ", " +
             BatchCount(ConvertShapeToLength(fShapeOutput)) + " * sizeof(*tensor_" + fNOutput + ")), \"Reshape\");\n";
   }
   // the same view on host pointers; the reference copies the elements (ROperator_Reshape.hxx Generate)
   std::string GenerateHost(std::string OpName) override
   {
      if (fShapeInput.empty()) throw std::runtime_error("TMVA SOFIE Reshape Op called to Generate without being initialized first");
      return "\n//------ " + std::string(fOpMode == Flatten ? "FLATTEN" : "RESHAPE") + " op_" + OpName + "\n" + SP +
             "if (static_cast<const void*>(tensor_" + fNOutput + ") != static_cast<const void*>(tensor_" + fNData +
             ")) std::memcpy(tensor_" + fNOutput + ", tensor_" + fNData + ", " + BatchCount(ConvertShapeToLength(fShapeOutput)) +
             " * sizeof(*tensor_" + fNOutput + "));\n";
   }
};

}   // namespace SOFIE
#endif
