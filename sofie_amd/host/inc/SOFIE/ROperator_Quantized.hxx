// Quantized and FP8 operators. The reference has none (its parser rejects int8 initialisers,
// src/SOFIE_parsers/src/RModelParser_ONNX.cxx:560-591, and Gemm/Conv accept float only,
// ROperator_Gemm.hxx:53-54, ROperator_Conv.hxx:61-66); these follow ONNX's QuantizeLinear,
// DequantizeLinear, QLinearMatMul and QLinearConv and plug into the same ROperator interface.
// Scales and zero-points must be initializers: they are folded at generation time into
//   - one fp32 scale per output channel, scale[n] = (s_in * s_w[n]) / s_out computed in fp32 in that order,
//   - one int32 bias per output channel, bias[n] - zp_in * sum_k w[k,n],
// which are the two vectors the kernels' fused requantisation reads.
#ifndef SOFIE_ROPERATOR_QUANTIZED
#define SOFIE_ROPERATOR_QUANTIZED

#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"
#include "SOFIE/ROperator_Conv.hxx"
#include "SOFIE/ROperator_Gemm.hxx"

namespace SOFIE {

namespace QUTIL {
inline float ScalarFloat(RModel &model, const std::string &name, const std::string &op)
{
   if (!model.IsInitializedTensor(name) || model.GetTensorType(name) != ETensorType::FLOAT ||
       ConvertShapeToLength(model.GetTensorShape(name)) != 1)
      throw std::runtime_error("TMVA SOFIE " + op + " Op: scale tensor " + name + " must be a float scalar initializer");
   return static_cast<float *>(model.GetInitializedTensorData(name).get())[0];
}
inline int ScalarZeroPoint(RModel &model, const std::string &name, const std::string &op)
{
   if (name.empty()) return 0;
   if (!model.IsInitializedTensor(name) || ConvertShapeToLength(model.GetTensorShape(name)) != 1)
      throw std::runtime_error("TMVA SOFIE " + op + " Op: zero-point tensor " + name + " must be a scalar initializer");
   void *p = model.GetInitializedTensorData(name).get();
   switch (model.GetTensorType(name)) {
   case ETensorType::INT8: return static_cast<int8_t *>(p)[0];
   case ETensorType::UINT8: return static_cast<uint8_t *>(p)[0];
   case ETensorType::INT32: return static_cast<int32_t *>(p)[0];
   default: throw std::runtime_error("TMVA SOFIE " + op + " Op: zero-point tensor " + name + " has an unsupported type");
   }
}
// per-channel float vector of length n from a scalar or [n] initializer
inline std::vector<float> ChannelScales(RModel &model, const std::string &name, size_t n, const std::string &op)
{
   if (!model.IsInitializedTensor(name) || model.GetTensorType(name) != ETensorType::FLOAT)
      throw std::runtime_error("TMVA SOFIE " + op + " Op: scale tensor " + name + " must be a float initializer");
   const size_t len = ConvertShapeToLength(model.GetTensorShape(name));
   if (len != 1 && len != n)
      throw std::runtime_error("TMVA SOFIE " + op + " Op: scale tensor " + name + " must have 1 or " + std::to_string(n) + " elements");
   const float *p = static_cast<float *>(model.GetInitializedTensorData(name).get());
   std::vector<float> v(n);
   for (size_t i = 0; i < n; ++i) v[i] = p[len == 1 ? 0 : i];
   return v;
}
inline void CheckSymmetricWeights(RModel &model, const std::string &zp, const std::string &op)
{
   if (zp.empty()) return;
   const size_t len = ConvertShapeToLength(model.GetTensorShape(zp));
   const int8_t *p = static_cast<int8_t *>(model.GetInitializedTensorData(zp).get());
   for (size_t i = 0; i < len; ++i)
      if (p[i] != 0) throw std::runtime_error("TMVA SOFIE " + op + " Op: weights must be symmetric (zero-point 0)");
}
template <class V> std::shared_ptr<void> Share(const std::vector<V> &v)
{
   std::shared_ptr<void> d(malloc(v.size() * sizeof(V) + 1), free);
   std::memcpy(d.get(), v.data(), v.size() * sizeof(V));
   return d;
}
inline void MarkFolded(RModel &model, const std::vector<std::string> &names)
{
   for (auto &n : names)
      if (!n.empty() && model.IsInitializedTensor(n)) model.SetNotWritableInitializedTensor(n);
}
}   // namespace QUTIL

// y = saturate_int8(round_half_even(x / scale) + zero_point)
class ROperator_QuantizeLinear final : public ROperator {
   std::string fNX, fNScale, fNZp, fNY;
   std::vector<size_t> fShape;
   float fScale = 1;
   int fZp = 0;
public:
   ROperator_QuantizeLinear(std::string nameX, std::string nameScale, std::string nameZp, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNScale(UTILITY::Clean_name(nameScale)), fNZp(UTILITY::Clean_name(nameZp)),
        fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "QuantizeLinear"; }
   // what a consumer needs to absorb this operator (valid after Initialize)
   const std::string &InputName() const { return fNX; }
   float Scale() const { return fScale; }
   int ZeroPoint() const { return fZp; }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType>) override { return {ETensorType::INT8}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override { return {input[0]}; }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE QuantizeLinear Op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("TMVA SOFIE QuantizeLinear Op Input Tensor " + fNX + " must be float");
      fShape = model.GetTensorShape(fNX);
      fScale = QUTIL::ScalarFloat(model, fNScale, "QuantizeLinear");
      fZp = QUTIL::ScalarZeroPoint(model, fNZp, "QuantizeLinear");
      if (!(fScale > 0)) throw std::runtime_error("TMVA SOFIE QuantizeLinear Op: scale must be positive");
      QUTIL::MarkFolded(model, {fNScale, fNZp});
      model.AddIntermediateTensor(fNY, ETensorType::INT8, fShape);
   }
   std::string Generate(std::string OpName) override
   {
      std::stringstream out;
      out << "\n//------ QuantizeLinear op_" << OpName << "\n";
      out << SP << "Check(sofie_hip_quantize_f32_s8(fCtx, tensor_" << fNX << ", tensor_" << fNY << ", " << BatchCount(ConvertShapeToLength(fShape))
          << ", " << FloatLiteral(fScale) << ", " << fZp << "), \"QuantizeLinear op_" << OpName << "\");\n";
      return out.str();
   }
   // host form: the definition, one element at a time (the division in fp32, as ONNX writes it)
   std::string GenerateHost(std::string OpName) override
   {
      std::stringstream out;
      out << "\n//------ QuantizeLinear op_" << OpName << "\n";
      out << SP << "for (size_t id = 0; id < " << BatchCount(ConvertShapeToLength(fShape)) << "; id++)\n";
      out << SP << SP << "tensor_" << fNY << "[id] = QuantizeOne(tensor_" << fNX << "[id], " << FloatLiteral(fScale) << ", " << fZp << ");\n";
      return out.str();
   }
};

// x = (q - zero_point) * scale
class ROperator_DequantizeLinear final : public ROperator {
   std::string fNX, fNScale, fNZp, fNY, fNXNchw;
   std::vector<size_t> fShape;
   float fScale = 1;
   int fZp = 0;
public:
   ROperator_DequantizeLinear(std::string nameX, std::string nameScale, std::string nameZp, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNScale(UTILITY::Clean_name(nameScale)), fNZp(UTILITY::Clean_name(nameZp)),
        fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "DequantizeLinear"; }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType>) override { return {ETensorType::FLOAT}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override { return {input[0]}; }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE DequantizeLinear Op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::INT8)
         throw std::runtime_error("TMVA SOFIE DequantizeLinear Op Input Tensor " + fNX + " must be int8");
      fShape = model.GetTensorShape(fNX);
      fScale = QUTIL::ScalarFloat(model, fNScale, "DequantizeLinear");
      fZp = QUTIL::ScalarZeroPoint(model, fNZp, "DequantizeLinear");
      QUTIL::MarkFolded(model, {fNScale, fNZp});
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShape);
      std::vector<size_t> chw;
      if (model.IsChannelsLast(fNX, &chw) && chw[0] > 1 && chw[1] * chw[2] > 1) {
         if (fShape.size() != 4)
            throw std::runtime_error("TMVA SOFIE DequantizeLinear Op: flattened channels-last tensor " + fNX + " cannot be dequantized");
         // float consumers expect [N,C,H,W]: convert the int8 tensor first
         fNXNchw = fNX + "_nchw";
         model.AddIntermediateTensor(fNXNchw, ETensorType::INT8, fShape);
         fOutputTensorNames.push_back(fNXNchw);
      }
   }
   std::string Generate(std::string OpName) override
   {
      std::stringstream out;
      out << "\n//------ DequantizeLinear op_" << OpName << "\n";
      std::string src = fNX;
      if (!fNXNchw.empty()) {
         out << SP << "Check(sofie_hip_relayout_s8(fCtx, tensor_" << fNX << ", tensor_" << fNXNchw << ", " << BatchCount(fShape[0]) << ", " << fShape[1]
             << ", " << fShape[2] << ", " << fShape[3] << ", SOFIE_LAYOUT_NHWC, SOFIE_LAYOUT_NCHW), \"DequantizeLinear op_" << OpName
             << "\");\n";
         src = fNXNchw;
      }
      out << SP << "Check(sofie_hip_dequantize_s8_f32(fCtx, tensor_" << src << ", tensor_" << fNY << ", " << BatchCount(ConvertShapeToLength(fShape))
          << ", " << FloatLiteral(fScale) << ", " << fZp << "), \"DequantizeLinear op_" << OpName << "\");\n";
      return out.str();
   }
   // host form: a channels-last tensor is read in its own order and written as [N,C,H,W]
   std::string GenerateHost(std::string OpName) override
   {
      std::stringstream out;
      out << "\n//------ DequantizeLinear op_" << OpName << "\n";
      if (!fNXNchw.empty()) {
         out << SP << "for (size_t n = 0; n < " << BatchCount(fShape[0]) << "; n++)\n";
         out << SP << SP << "for (size_t c = 0; c < " << fShape[1] << "; c++)\n";
         out << SP << SP << SP << "for (size_t p = 0; p < " << fShape[2] * fShape[3] << "; p++)\n";
         out << SP << SP << SP << SP << "tensor_" << fNY << "[(n * " << fShape[1] << " + c) * " << fShape[2] * fShape[3]
             << " + p] = static_cast<float>(static_cast<int>(tensor_" << fNX << "[(n * " << fShape[2] * fShape[3] << " + p) * " << fShape[1]
             << " + c]) - (" << fZp << ")) * " << FloatLiteral(fScale) << ";\n";
         return out.str();
      }
      out << SP << "for (size_t id = 0; id < " << BatchCount(ConvertShapeToLength(fShape)) << "; id++)\n";
      out << SP << SP << "tensor_" << fNY << "[id] = static_cast<float>(static_cast<int>(tensor_" << fNX << "[id]) - (" << fZp << ")) * "
          << FloatLiteral(fScale) << ";\n";
      return out.str();
   }
};

// QLinearMatMul with an optional int32 bias (ONNX QLinearMatMul inputs a, a_scale, a_zero_point, b, b_scale,
// b_zero_point, y_scale, y_zero_point; the bias follows the QGemm convention: int32, scale a_scale*b_scale).
// B must be an initializer: it is transposed once at generation time into the K-contiguous [N,K] layout.
// An empty nameYScale selects fp32 output y = float(acc + bias) * (a_scale * b_scale[n]).
class ROperator_QLinearMatMul final : public ROperator {
   std::string fNA, fNAScale, fNAZp, fNB, fNBScale, fNBZp, fNYScale, fNYZp, fNBias, fNY;
   std::string fNBt, fNScale, fNQBias;
   int_t fTransB = 0;
   std::vector<size_t> fShapeA, fShapeB;
   size_t fM = 0, fN = 0, fK = 0;
   int fZpY = 0;
   bool fFloatOut = false, fHasBias = false;
   EActivationType fActivation = EActivationType::UNDEFINED;
   // the narrow layer that follows this one, emitted with it as one call (RModel::FuseQLinearPair)
   struct Tail {
      std::string weights, scale, bias, out;
      size_t N = 0;
      int zpY = 0;
      bool relu = false, floatOut = false;
   };
   bool fHasTail = false;
   Tail fTail;
public:
   // --- pairs of layers -------------------------------------------------------------------------------------
   const std::string &NameA() const { return fNA; }
   const std::string &NameY() const { return fNY; }
   size_t Columns() const { return fN; }
   size_t Depth() const { return fK; }
   bool FloatOut() const { return fFloatOut; }
   bool HasTail() const { return fHasTail; }
   // this operator as the second layer of a pair
   Tail AsTail() const
   {
      Tail t;
      t.weights = fNBt;
      t.scale = fNScale;
      t.bias = fHasBias ? fNQBias : "";
      t.out = fNY;
      t.N = fN;
      t.zpY = fZpY;
      t.relu = fActivation == EActivationType::RELU;
      t.floatOut = fFloatOut;
      return t;
   }
   // This operator writes the second layer's output as well; its own output stays in the pool as the tensor the
   // library may use between the layers.
   void AppendTail(const Tail &t)
   {
      fHasTail = true;
      fTail = t;
      fOutputTensorNames = {fNY, t.out};
      fInputTensorNames.push_back(t.weights);
      fInputTensorNames.push_back(t.scale);
      if (!t.bias.empty()) fInputTensorNames.push_back(t.bias);
   }
   ROperator_QLinearMatMul(std::string nameA, std::string nameAScale, std::string nameAZp, std::string nameB,
                           std::string nameBScale, std::string nameBZp, std::string nameYScale, std::string nameYZp,
                           std::string nameY, std::string nameBias = "", int_t transB = 0)
      : fNA(UTILITY::Clean_name(nameA)), fNAScale(UTILITY::Clean_name(nameAScale)), fNAZp(UTILITY::Clean_name(nameAZp)),
        fNB(UTILITY::Clean_name(nameB)), fNBScale(UTILITY::Clean_name(nameBScale)), fNBZp(UTILITY::Clean_name(nameBZp)),
        fNYScale(UTILITY::Clean_name(nameYScale)), fNYZp(UTILITY::Clean_name(nameYZp)), fNBias(UTILITY::Clean_name(nameBias)),
        fNY(UTILITY::Clean_name(nameY)), fTransB(transB)
   {
      fFloatOut = fNYScale.empty();
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "QLinearMatMul"; }
   bool FuseActivation(EActivationType act) override
   {
      if (act != EActivationType::RELU || fActivation != EActivationType::UNDEFINED) return false;
      fActivation = act;
      return true;
   }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType>) override
   {
      return {fFloatOut ? ETensorType::FLOAT : ETensorType::INT8};
   }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      std::vector<size_t> b = input[1];
      if (fTransB) std::reverse(b.begin(), b.end());
      return {{input[0][0], b[1]}};
   }
   void Initialize(RModel &model) override
   {
      const std::string op = "QLinearMatMul";
      if (!model.CheckIfTensorAlreadyExist(fNA) || !model.CheckIfTensorAlreadyExist(fNB))
         throw std::runtime_error("TMVA SOFIE QLinearMatMul Op Input Tensor " + fNA + " or " + fNB + " is not found in model");
      if (model.GetTensorType(fNA) != ETensorType::INT8 || model.GetTensorType(fNB) != ETensorType::INT8)
         throw std::runtime_error("TMVA SOFIE QLinearMatMul Op: A and B must be int8 tensors");
      if (!model.IsInitializedTensor(fNB))
         throw std::runtime_error("TMVA SOFIE QLinearMatMul Op: B (" + fNB + ") must be an initializer");
      fShapeA = model.GetTensorShape(fNA);
      fShapeB = model.GetTensorShape(fNB);
      if (fShapeA.size() != 2 || fShapeB.size() != 2)
         throw std::runtime_error("TMVA SOFIE QLinearMatMul Op: only rank-2 operands are supported");
      fM = fShapeA[0];
      fK = fShapeA[1];
      fN = fTransB ? fShapeB[0] : fShapeB[1];
      if ((fTransB ? fShapeB[1] : fShapeB[0]) != fK)
         throw std::runtime_error("TMVA SOFIE QLinearMatMul Op " + fNY + " has invalid shape" + ConvertShapeToString(fShapeA) + " x " +
                                  ConvertShapeToString(fShapeB));
      const float sa = QUTIL::ScalarFloat(model, fNAScale, op);
      const int zpa = QUTIL::ScalarZeroPoint(model, fNAZp, op);
      const std::vector<float> sb = QUTIL::ChannelScales(model, fNBScale, fN, op);
      QUTIL::CheckSymmetricWeights(model, fNBZp, op);
      const float sy = fFloatOut ? 1.0f : QUTIL::ScalarFloat(model, fNYScale, op);
      fZpY = fFloatOut ? 0 : QUTIL::ScalarZeroPoint(model, fNYZp, op);
      // weights: [N,K], K contiguous
      // If A is the Flatten of a channels-last tensor its columns are in (h,w,c) order: the weight rows
      // are permuted to that order here instead of moving the activations at run time.
      std::vector<size_t> chw;
      const bool permute = model.IsChannelsLast(fNA, &chw) && chw[0] > 1 && chw[1] * chw[2] > 1;
      if (permute && chw[0] * chw[1] * chw[2] != fK)
         throw std::runtime_error("TMVA SOFIE QLinearMatMul Op: channels-last input " + fNA + " does not match K");
      const int8_t *b = static_cast<int8_t *>(model.GetInitializedTensorData(fNB).get());
      std::vector<int8_t> bt(fN * fK);
      std::vector<int64_t> colsum(fN, 0);
      for (size_t k = 0; k < fK; ++k) {
         size_t kdst = k;
         if (permute) {
            const size_t hw = chw[1] * chw[2], c = k / hw, pos = k % hw;
            kdst = pos * chw[0] + c;
         }
         for (size_t n = 0; n < fN; ++n) {
            const int8_t v = fTransB ? b[n * fK + k] : b[k * fN + n];
            bt[n * fK + kdst] = v;
            colsum[n] += v;
         }
      }
      fNBt = fNB + (permute ? "_nk_cl" : "_nk");
      if (!model.CheckIfTensorAlreadyExist(fNBt)) model.AddInitializedTensor(fNBt, ETensorType::INT8, {fN, fK}, QUTIL::Share(bt));
      // per-column scale
      std::vector<float> scale(fN);
      for (size_t n = 0; n < fN; ++n) {
         const float prod = sa * sb[n];
         scale[n] = fFloatOut ? prod : prod / sy;
      }
      fNScale = fNY + "_qscale";
      model.AddInitializedTensor(fNScale, ETensorType::FLOAT, {fN}, QUTIL::Share(scale));
      // int32 bias with the activation zero-point folded in
      fHasBias = !fNBias.empty() || zpa != 0;
      if (fHasBias) {
         std::vector<int32_t> qb(fN, 0);
         if (!fNBias.empty()) {
            if (!model.IsInitializedTensor(fNBias) || model.GetTensorType(fNBias) != ETensorType::INT32 ||
                ConvertShapeToLength(model.GetTensorShape(fNBias)) != fN)
               throw std::runtime_error("TMVA SOFIE QLinearMatMul Op: bias " + fNBias + " must be an int32 initializer of length N");
            const int32_t *pb = static_cast<int32_t *>(model.GetInitializedTensorData(fNBias).get());
            for (size_t n = 0; n < fN; ++n) qb[n] = pb[n];
         }
         for (size_t n = 0; n < fN; ++n) qb[n] = (int32_t)((int64_t)qb[n] - (int64_t)zpa * colsum[n]);
         fNQBias = fNY + "_qbias";
         model.AddInitializedTensor(fNQBias, ETensorType::INT32, {fN}, QUTIL::Share(qb));
      }
      QUTIL::MarkFolded(model, {fNB, fNAScale, fNAZp, fNBScale, fNBZp, fNYScale, fNYZp, fNBias});
      fInputTensorNames = {fNA, fNBt, fNScale};
      if (fHasBias) fInputTensorNames.push_back(fNQBias);
      model.AddIntermediateTensor(fNY, fFloatOut ? ETensorType::FLOAT : ETensorType::INT8, std::vector<size_t>{fM, fN});
   }
   std::string Generate(std::string OpName) override
   {
      if (fShapeA.empty()) throw std::runtime_error("TMVA SOFIE QLinearMatMul Op called to Generate without being initialized first");
      std::stringstream out;
      if (fHasTail) {
         out << "\n//--------- QLinearMatMul x 2 op_" << OpName << " (the second layer in the same call)\n";
         out << SP << "Check(sofie_hip_qgemm_s8_pair(fCtx, " << BatchCount(fM) << ", " << fK << ", tensor_" << fNA << ", " << fK << ", "
             << fN << ", tensor_" << fNBt << ", " << fK << ", tensor_" << fNScale << ", "
             << (fHasBias ? "tensor_" + fNQBias : std::string("nullptr")) << ", " << fZpY << ", "
             << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << ", tensor_" << fNY << ", " << fN << ", "
             << fTail.N << ", tensor_" << fTail.weights << ", " << fN << ", tensor_" << fTail.scale << ", "
             << (fTail.bias.empty() ? std::string("nullptr") : "tensor_" + fTail.bias) << ", " << fTail.zpY << ", "
             << (fTail.relu ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << ", tensor_" << fTail.out << ", " << fTail.N << ", "
             << (fTail.floatOut ? "SOFIE_OUT_F32" : "SOFIE_OUT_S8") << "), \"QLinearMatMul pair op_" << OpName << "\");\n";
         return out.str();
      }
      out << "\n//--------- QLinearMatMul op_" << OpName << "\n";
      out << SP << "Check(sofie_hip_qgemm_s8(fCtx, 1, " << BatchCount(fM) << ", " << fN << ", " << fK << ", tensor_" << fNA << ", " << fK
          << ", tensor_" << fNBt << ", " << fK << ", tensor_" << fNScale << ", "
          << (fHasBias ? "tensor_" + fNQBias : std::string("nullptr")) << ", " << fZpY << ", "
          << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << ", tensor_" << fNY << ", " << fN << ", "
          << (fFloatOut ? "SOFIE_OUT_F32" : "SOFIE_OUT_S8") << "), \"QLinearMatMul op_" << OpName << "\");\n";
      return out.str();
   }
   // host form: int32 sums over the [N,K] weights packed at generation time, then the requantisation (or, for a float
   // output, the accumulator times the scale), one output at a time
   std::string GenerateHost(std::string OpName) override
   {
      if (fShapeA.empty()) throw std::runtime_error("TMVA SOFIE QLinearMatMul Op called to Generate without being initialized first");
      if (fHasTail) throw std::runtime_error("TMVA SOFIE QLinearMatMul Op: a pair of layers has no host emission");
      const std::string relu = fActivation == EActivationType::RELU ? "true" : "false";
      std::stringstream out;
      out << "\n//--------- QLinearMatMul op_" << OpName << "\n";
      out << SP << "for (size_t m = 0; m < " << BatchCount(fM) << "; m++) {\n";
      out << SP << SP << "const int8_t * a = tensor_" << fNA << " + m * " << fK << ";\n";
      out << SP << SP << "for (size_t n = 0; n < " << fN << "; n++) {\n";
      out << SP << SP << SP << "const int8_t * b = tensor_" << fNBt << " + n * " << fK << ";\n";
      out << SP << SP << SP << "int32_t acc = " << (fHasBias ? "tensor_" + fNQBias + "[n]" : std::string("0")) << ";\n";
      out << SP << SP << SP << "for (size_t k = 0; k < " << fK << "; k++) acc += static_cast<int32_t>(a[k]) * static_cast<int32_t>(b[k]);\n";
      if (fFloatOut) {
         out << SP << SP << SP << "float v = static_cast<float>(acc) * tensor_" << fNScale << "[n];\n";
         if (fActivation == EActivationType::RELU) out << SP << SP << SP << "if (!(v > 0)) v = 0;\n";
         out << SP << SP << SP << "tensor_" << fNY << "[m * " << fN << " + n] = v;\n";
      } else {
         out << SP << SP << SP << "tensor_" << fNY << "[m * " << fN << " + n] = Requantize(acc, tensor_" << fNScale << "[n], " << fZpY << ", "
             << relu << ");\n";
      }
      out << SP << SP << "}\n";
      out << SP << "}\n";
      return out.str();
   }
};

// QLinearConv (2-D): x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, optional int32 bias.
// Geometry attributes and their defaults are those of ROperator_Conv.
class ROperator_QLinearConv final : public ROperator {
   ConvGeometry fGeom;
   std::string fNX, fNXScale, fNXZp, fNW, fNWScale, fNWZp, fNYScale, fNYZp, fNBias, fNY;
   std::string fNScale, fNQBias, fNWPacked, fNYPooled, fNXFloat;
   float fScaleX = 0;
   std::vector<size_t> fShapeX, fShapeW, fShapeY, fShapePooled, fPoolKernel, fPoolStrides;
   int fZpX = 0, fZpY = 0;
   bool fHasBias = false, fXChannelsLast = false;
   EActivationType fActivation = EActivationType::UNDEFINED;
   // the layers that follow this one in the same library call (RModel::FuseQLinearConvChain): their descriptors, printed
   std::vector<std::string> fChain;
public:
   // --- chains of layers: this operator and the QLinearConv operators that read its output, one after the other, are
   // emitted as one sofie_hip_qconv2d_s8_chain call, which runs two of them in one launch where the batch allows it
   const std::string &OutputName() const { return fPoolKernel.empty() ? fNY : fNYPooled; }
   const std::string &InputName() const { return fNX; }
   bool ChainHead() const { return fNXFloat.empty() && fXChannelsLast && !fShapeX.empty(); }
   bool ChainLayer() const { return ChainHead() && fChain.empty(); }
   size_t ChainLength() const { return 1 + fChain.size(); }
   // one initializer of a sofie_hip_qconv_layer
   std::string LayerDescriptor()
   {
      size_t pt, pl, pb, pr;
      fGeom.Pads2D(pt, pl, pb, pr);
      const bool pooled = !fPoolKernel.empty();
      std::stringstream d;
      d << "{tensor_" << fNWPacked << ", SOFIE_LAYOUT_NHWC, " << (fHasBias ? "tensor_" + fNQBias : std::string("nullptr")) << ", tensor_"
        << fNScale << ", tensor_" << OutputName() << ", SOFIE_LAYOUT_NHWC, " << fShapeX[1] << ", " << fShapeX[2] << ", " << fShapeX[3]
        << ", " << fShapeW[0] << ", " << fShapeW[2] << ", " << fShapeW[3] << ", " << pt << ", " << pl << ", " << pb << ", " << pr << ", "
        << fGeom.strides[0] << ", " << fGeom.strides[1] << ", " << fGeom.group << ", " << fZpX << ", " << fZpY << ", "
        << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE") << ", ";
      if (pooled) d << fPoolKernel[0] << ", " << fPoolKernel[1] << ", " << fPoolStrides[0] << ", " << fPoolStrides[1];
      else d << "0, 0, 0, 0";
      d << "}";
      return d.str();
   }
   void AppendLayer(ROperator_QLinearConv &next)
   {
      fChain.push_back(next.LayerDescriptor());
      fOutputTensorNames.push_back(next.OutputName());
      for (auto &n : next.GetOpInputTensors())
         if (n != next.InputName()) fInputTensorNames.push_back(n);
   }
   ROperator_QLinearConv(std::string autopad, std::vector<size_t> dilations, size_t group, std::vector<size_t> kernelShape,
                         std::vector<size_t> pads, std::vector<size_t> strides, std::string nameX, std::string nameXScale,
                         std::string nameXZp, std::string nameW, std::string nameWScale, std::string nameWZp,
                         std::string nameYScale, std::string nameYZp, std::string nameBias, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNXScale(UTILITY::Clean_name(nameXScale)), fNXZp(UTILITY::Clean_name(nameXZp)),
        fNW(UTILITY::Clean_name(nameW)), fNWScale(UTILITY::Clean_name(nameWScale)), fNWZp(UTILITY::Clean_name(nameWZp)),
        fNYScale(UTILITY::Clean_name(nameYScale)), fNYZp(UTILITY::Clean_name(nameYZp)), fNBias(UTILITY::Clean_name(nameBias)),
        fNY(UTILITY::Clean_name(nameY))
   {
      fGeom.autopad = autopad; fGeom.dilations = dilations; fGeom.group = group; fGeom.kernel = kernelShape;
      fGeom.pads = pads; fGeom.strides = strides;
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "QLinearConv"; }
   bool FuseActivation(EActivationType act) override
   {
      if (act != EActivationType::RELU || fActivation != EActivationType::UNDEFINED) return false;
      fActivation = act;
      return true;
   }
   bool FuseInputQuantization(const std::string &xFloat, float scale, int zeroPoint) override
   {
      // the fused call exists for any shape, but only first layers (one input channel, 3x3, stride 1, pad 1,
      // OC a multiple of 16) have a kernel that never writes the int8 input: fuse only those
      if (fShapeX.empty() || !fNXFloat.empty() || fXChannelsLast) return false;
      size_t pt, pl, pb, pr;
      fGeom.Pads2D(pt, pl, pb, pr);
      if (fShapeX[1] != 1 || fGeom.group != 1 || fShapeW[2] != 3 || fShapeW[3] != 3 || fGeom.strides[0] != 1 ||
          fGeom.strides[1] != 1 || pt != 1 || pl != 1 || pb != 1 || pr != 1 || fShapeW[0] % 16 != 0)
         return false;
      if (zeroPoint != fZpX || scale != fScaleX) return false;   // must be the quantization this operator assumes
      fNXFloat = xFloat;
      for (auto &n : fInputTensorNames)
         if (n == fNX) n = xFloat;
      return true;
   }
   bool FusePooling(const std::vector<size_t> &kernel, const std::vector<size_t> &strides, const std::string &pooledName,
                    const std::vector<size_t> &pooledShape) override
   {
      if (fShapeY.empty() || !fPoolKernel.empty() || kernel.size() != 2 || strides.size() != 2) return false;
      if (kernel[0] > fShapeY[2] || kernel[1] > fShapeY[3]) return false;
      fPoolKernel = kernel;
      fPoolStrides = strides;
      fNYPooled = pooledName;
      fShapePooled = pooledShape;
      fOutputTensorNames = {fNYPooled};
      return true;
   }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType>) override { return {ETensorType::INT8}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      return {fGeom.Resolve(input[0], input[1])};
   }
   void Initialize(RModel &model) override
   {
      const std::string op = "QLinearConv";
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("TMVA SOFIE QLinearConv op Input Tensor " + fNX + " is not found in model");
      if (!model.IsInitializedTensor(fNW))
         throw std::runtime_error("TMVA SOFIE QLinearConv op weight Tensor " + fNW + " must be an initializer");
      if (model.GetTensorType(fNX) != ETensorType::INT8 || model.GetTensorType(fNW) != ETensorType::INT8)
         throw std::runtime_error("TMVA SOFIE QLinearConv Op: x and w must be int8 tensors");
      fShapeX = model.GetTensorShape(fNX);
      fShapeW = model.GetTensorShape(fNW);
      if (fShapeX.size() != 4 || fShapeW.size() != 4)
         throw std::runtime_error("TMVA SOFIE QLinearConv Op: only 2-D convolutions (4-D tensors) are supported");
      fShapeY = ShapeInference({fShapeX, fShapeW})[0];
      for (auto d : fGeom.dilations)
         if (d != 1) throw std::runtime_error("TMVA SOFIE QLinearConv Op: dilations are not supported");
      if (fShapeW[1] * fGeom.group != fShapeX[1])
         throw std::runtime_error("TMVA SOFIE QLinearConv op: weight tensor " + fNW + " does not match the input channels and group");
      const size_t OC = fShapeW[0], per = fShapeW[1] * fShapeW[2] * fShapeW[3];
      const float sx = QUTIL::ScalarFloat(model, fNXScale, op);
      fScaleX = sx;
      fZpX = QUTIL::ScalarZeroPoint(model, fNXZp, op);
      const std::vector<float> sw = QUTIL::ChannelScales(model, fNWScale, OC, op);
      QUTIL::CheckSymmetricWeights(model, fNWZp, op);
      const float sy = QUTIL::ScalarFloat(model, fNYScale, op);
      fZpY = QUTIL::ScalarZeroPoint(model, fNYZp, op);
      std::vector<float> scale(OC);
      for (size_t oc = 0; oc < OC; ++oc) scale[oc] = (sx * sw[oc]) / sy;
      fNScale = fNY + "_qscale";
      model.AddInitializedTensor(fNScale, ETensorType::FLOAT, {OC}, QUTIL::Share(scale));
      fHasBias = !fNBias.empty() || fZpX != 0;
      if (fHasBias) {
         const int8_t *w = static_cast<int8_t *>(model.GetInitializedTensorData(fNW).get());
         std::vector<int32_t> qb(OC, 0);
         if (!fNBias.empty()) {
            if (!model.IsInitializedTensor(fNBias) || model.GetTensorType(fNBias) != ETensorType::INT32 ||
                ConvertShapeToLength(model.GetTensorShape(fNBias)) != OC)
               throw std::runtime_error("TMVA SOFIE QLinearConv op: Bias Tensor has wrong shape: " +
                                        ConvertShapeToString(model.GetTensorShape(fNBias)));
            const int32_t *pb = static_cast<int32_t *>(model.GetInitializedTensorData(fNBias).get());
            for (size_t oc = 0; oc < OC; ++oc) qb[oc] = pb[oc];
         }
         for (size_t oc = 0; oc < OC; ++oc) {
            int64_t s = 0;
            for (size_t i = 0; i < per; ++i) s += w[oc * per + i];
            qb[oc] = (int32_t)((int64_t)qb[oc] - (int64_t)fZpX * s);
         }
         fNQBias = fNY + "_qbias";
         model.AddInitializedTensor(fNQBias, ETensorType::INT32, {OC}, QUTIL::Share(qb));
      }
      QUTIL::MarkFolded(model, {fNXScale, fNXZp, fNWScale, fNWZp, fNYScale, fNYZp, fNBias});
      // Layouts: the output is kept channels-last (what the matrix-core kernel writes and what the next
      // quantized operator reads); the weights are repacked once, here, to [OC][KH][KW][C/group].
      fXChannelsLast = model.IsChannelsLast(fNX);
      model.MarkChannelsLast(fNY, fShapeY[1], fShapeY[2], fShapeY[3]);
      {
         const int8_t *w = static_cast<int8_t *>(model.GetInitializedTensorData(fNW).get());
         const size_t icg = fShapeW[1], khw = fShapeW[2] * fShapeW[3];
         std::vector<int8_t> packed(OC * per);
         for (size_t oc = 0; oc < OC; ++oc)
            for (size_t ic = 0; ic < icg; ++ic)
               for (size_t t = 0; t < khw; ++t) packed[(oc * khw + t) * icg + ic] = w[(oc * icg + ic) * khw + t];
         fNWPacked = fNW + "_ohwi";
         if (!model.CheckIfTensorAlreadyExist(fNWPacked))
            model.AddInitializedTensor(fNWPacked, ETensorType::INT8, {OC, fShapeW[2], fShapeW[3], icg}, QUTIL::Share(packed));
         QUTIL::MarkFolded(model, {fNW});
      }
      fInputTensorNames = {fNX, fNWPacked, fNScale};
      if (fHasBias) fInputTensorNames.push_back(fNQBias);
      model.AddIntermediateTensor(fNY, ETensorType::INT8, fShapeY);
   }
   std::string Generate(std::string OpName) override
   {
      if (fShapeX.empty()) throw std::runtime_error("TMVA SOFIE QLinearConv Op called to Generate without being initialized first");
      size_t pt, pl, pb, pr;
      fGeom.Pads2D(pt, pl, pb, pr);
      std::stringstream out;
      const bool pooled = !fPoolKernel.empty();
      const bool fromFloat = !fNXFloat.empty();
      if (!fChain.empty()) {
         out << "\n//----  operator QLinearConv x " << ChainLength() << " op_" << OpName << " (the layers behind it in the same call)\n";
         out << SP << "{\n";
         out << SP << SP << "const sofie_hip_qconv_layer layers[" << ChainLength() << "] = {\n";
         out << SP << SP << SP << LayerDescriptor();
         for (auto &d : fChain) out << ",\n" << SP << SP << SP << d;
         out << "};\n";
         out << SP << SP << "Check(sofie_hip_qconv2d_s8_chain(fCtx, tensor_" << fNX << ", SOFIE_LAYOUT_NHWC, " << BatchCount(fShapeX[0])
             << ", " << ChainLength() << ", layers), \"QLinearConv chain op_" << OpName << "\");\n";
         out << SP << "}\n";
         return out.str();
      }
      out << "\n//----  operator " << (fromFloat ? "QuantizeLinear + " : "") << "QLinearConv" << (pooled ? " + MaxPool" : "") << " op_"
          << OpName << "\n";
      out << SP << "Check(";
      if (fromFloat)
         out << "sofie_hip_quantize_qconv2d_s8(fCtx, tensor_" << fNXFloat << ", " << FloatLiteral(fScaleX) << ", " << fZpX;
      else
         out << (pooled ? "sofie_hip_qconv2d_pool_s8" : "sofie_hip_qconv2d_s8") << "(fCtx, tensor_" << fNX << ", "
             << (fXChannelsLast ? "SOFIE_LAYOUT_NHWC" : "SOFIE_LAYOUT_NCHW");
      out << ", tensor_" << fNWPacked << ", SOFIE_LAYOUT_NHWC, " << (fHasBias ? "tensor_" + fNQBias : std::string("nullptr"))
          << ", tensor_" << fNScale << ", tensor_" << (pooled ? fNYPooled : fNY) << ", SOFIE_LAYOUT_NHWC, " << BatchCount(fShapeX[0]) << ", "
          << fShapeX[1] << ", " << fShapeX[2] << ", " << fShapeX[3] << ", " << fShapeW[0] << ", " << fShapeW[2] << ", " << fShapeW[3]
          << ", " << pt << ", " << pl << ", " << pb << ", " << pr << ", " << fGeom.strides[0] << ", " << fGeom.strides[1] << ", " << fGeom.group << ", ";
      if (!fromFloat) out << fZpX << ", ";
      out << fZpY << ", " << (fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE");
      if (pooled)
         out << ", " << fPoolKernel[0] << ", " << fPoolKernel[1] << ", " << fPoolStrides[0] << ", " << fPoolStrides[1];
      else if (fromFloat)
         out << ", 0, 0, 0, 0";
      else
         out << ", SOFIE_OUT_S8";
      out << "), \"QLinearConv op_" << OpName << "\");\n";
      return out.str();
   }
   // host form: the definition on the tensors as the generated code keeps them (input channels-last or [N,C,H,W],
   // weights [OC][KH][KW][C/group], output channels-last): an int32 sum per output over the window, cells outside the
   // image counting as the input zero-point (which the folded bias takes out again), then the requantisation
   std::string GenerateHost(std::string OpName) override
   {
      if (fShapeX.empty()) throw std::runtime_error("TMVA SOFIE QLinearConv Op called to Generate without being initialized first");
      if (!fChain.empty() || !fPoolKernel.empty() || !fNXFloat.empty())
         throw std::runtime_error("TMVA SOFIE QLinearConv Op: fused layers have no host emission");
      size_t pt, pl, pb, pr;
      fGeom.Pads2D(pt, pl, pb, pr);
      const size_t C = fShapeX[1], H = fShapeX[2], W = fShapeX[3], OC = fShapeW[0], Cg = fShapeW[1], KH = fShapeW[2], KW = fShapeW[3];
      const size_t OH = fShapeY[2], OW = fShapeY[3], OCg = OC / fGeom.group;
      std::stringstream out;
      out << "\n//----  operator QLinearConv op_" << OpName << "\n";
      out << SP << "for (size_t n = 0; n < " << BatchCount(fShapeX[0]) << "; n++)\n";
      out << SP << " for (size_t oh = 0; oh < " << OH << "; oh++)\n";
      out << SP << "  for (size_t ow = 0; ow < " << OW << "; ow++)\n";
      out << SP << "   for (size_t oc = 0; oc < " << OC << "; oc++) {\n";
      out << SP << SP << "const size_t c0 = (oc / " << OCg << ") * " << Cg << ";\n";
      out << SP << SP << "int32_t acc = " << (fHasBias ? "tensor_" + fNQBias + "[oc]" : std::string("0")) << ";\n";
      out << SP << SP << "for (size_t kh = 0; kh < " << KH << "; kh++)\n";
      out << SP << SP << " for (size_t kw = 0; kw < " << KW << "; kw++) {\n";
      out << SP << SP << SP << "const long ih = static_cast<long>(oh * " << fGeom.strides[0] << " + kh) - " << pt << ", iw = static_cast<long>(ow * "
          << fGeom.strides[1] << " + kw) - " << pl << ";\n";
      out << SP << SP << SP << "const bool inside = ih >= 0 && ih < " << H << " && iw >= 0 && iw < " << W << ";\n";
      out << SP << SP << SP << "const int8_t * w = tensor_" << fNWPacked << " + ((oc * " << KH << " + kh) * " << KW << " + kw) * " << Cg << ";\n";
      out << SP << SP << SP << "for (size_t ic = 0; ic < " << Cg << "; ic++) {\n";
      if (fXChannelsLast)
         out << SP << SP << SP << SP << "const int32_t x = inside ? tensor_" << fNX << "[((n * " << H << " + ih) * " << W << " + iw) * " << C
             << " + c0 + ic] : " << fZpX << ";\n";
      else
         out << SP << SP << SP << SP << "const int32_t x = inside ? tensor_" << fNX << "[((n * " << C << " + c0 + ic) * " << H << " + ih) * " << W
             << " + iw] : " << fZpX << ";\n";
      out << SP << SP << SP << SP << "acc += x * static_cast<int32_t>(w[ic]);\n";
      out << SP << SP << SP << "}\n";
      out << SP << SP << " }\n";
      out << SP << SP << "tensor_" << fNY << "[((n * " << OH << " + oh) * " << OW << " + ow) * " << OC << " + oc] = Requantize(acc, tensor_"
          << fNScale << "[oc], " << fZpY << ", " << (fActivation == EActivationType::RELU ? "true" : "false") << ");\n";
      out << SP << "   }\n";
      return out.str();
   }
};

// FP8 e4m3 GEMM: Y = bf16( (A x B) * (scale_a*scale_b) + bias ). A is an e4m3 tensor (FLOAT8E4M3FN), B an e4m3
// initializer [K,N] (transposed once at generation time) or [N,K] with transB; scales are float scalar initializers.
class ROperator_GemmFP8 final : public ROperator {
   std::string fNA, fNB, fNAScale, fNBScale, fNBias, fNY, fNBt;
   int_t fTransB = 0;
   size_t fM = 0, fN = 0, fK = 0;
   float fSa = 1, fSb = 1;
public:
   ROperator_GemmFP8(std::string nameA, std::string nameAScale, std::string nameB, std::string nameBScale, std::string nameBias,
                     std::string nameY, int_t transB = 0)
      : fNA(UTILITY::Clean_name(nameA)), fNB(UTILITY::Clean_name(nameB)), fNAScale(UTILITY::Clean_name(nameAScale)),
        fNBScale(UTILITY::Clean_name(nameBScale)), fNBias(UTILITY::Clean_name(nameBias)), fNY(UTILITY::Clean_name(nameY)),
        fTransB(transB)
   {
      fOutputTensorNames = {fNY};
   }
   std::string Kind() const override { return "GemmFP8"; }
   std::vector<ETensorType> TypeInference(std::vector<ETensorType>) override { return {ETensorType::BFLOAT16}; }
   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      std::vector<size_t> b = input[1];
      if (fTransB) std::reverse(b.begin(), b.end());
      return {{input[0][0], b[1]}};
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNA) || !model.IsInitializedTensor(fNB))
         throw std::runtime_error("TMVA SOFIE GemmFP8 Op Input Tensor " + fNA + " or initializer " + fNB + " is not found in model");
      if (model.GetTensorType(fNA) != ETensorType::FLOAT8E4M3FN || model.GetTensorType(fNB) != ETensorType::FLOAT8E4M3FN)
         throw std::runtime_error("TMVA SOFIE GemmFP8 Op: A and B must be e4m3 tensors");
      auto sa = model.GetTensorShape(fNA), sb = model.GetTensorShape(fNB);
      if (sa.size() != 2 || sb.size() != 2) throw std::runtime_error("TMVA SOFIE GemmFP8 Op: only rank-2 operands are supported");
      fM = sa[0]; fK = sa[1];
      fN = fTransB ? sb[0] : sb[1];
      if ((fTransB ? sb[1] : sb[0]) != fK) throw std::runtime_error("TMVA SOFIE GemmFP8 Op " + fNY + " has invalid shape");
      fSa = QUTIL::ScalarFloat(model, fNAScale, "GemmFP8");
      fSb = QUTIL::ScalarFloat(model, fNBScale, "GemmFP8");
      const uint8_t *b = static_cast<uint8_t *>(model.GetInitializedTensorData(fNB).get());
      std::vector<uint8_t> bt(fN * fK);
      for (size_t k = 0; k < fK; ++k)
         for (size_t n = 0; n < fN; ++n) bt[n * fK + k] = fTransB ? b[n * fK + k] : b[k * fN + n];
      fNBt = fNB + "_nk";
      if (!model.CheckIfTensorAlreadyExist(fNBt))
         model.AddInitializedTensor(fNBt, ETensorType::FLOAT8E4M3FN, {fN, fK}, QUTIL::Share(bt));
      QUTIL::MarkFolded(model, {fNB, fNAScale, fNBScale});
      fInputTensorNames = {fNA, fNBt};
      if (!fNBias.empty()) {
         if (!model.CheckIfTensorAlreadyExist(fNBias) || ConvertShapeToLength(model.GetTensorShape(fNBias)) != fN)
            throw std::runtime_error("TMVA SOFIE GemmFP8 Op: bias " + fNBias + " must have N elements");
         fInputTensorNames.push_back(fNBias);
      }
      model.AddIntermediateTensor(fNY, ETensorType::BFLOAT16, std::vector<size_t>{fM, fN});
   }
   std::string Generate(std::string OpName) override
   {
      std::stringstream out;
      out << "\n//--------- GemmFP8 op_" << OpName << "\n";
      out << SP << "Check(sofie_hip_gemm_fp8(fCtx, 1, " << BatchCount(fM) << ", " << fN << ", " << fK << ", tensor_" << fNA << ", " << fK
          << ", tensor_" << fNBt << ", " << fK << ", " << FloatLiteral(fSa) << ", " << FloatLiteral(fSb) << ", "
          << (fNBias.empty() ? std::string("nullptr") : "tensor_" + fNBias) << ", tensor_" << fNY << ", " << fN
          << ", SOFIE_OUT_BF16), \"GemmFP8 op_" << OpName << "\");\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
