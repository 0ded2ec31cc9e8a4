// Gemm / MatMul(+Add) / Gemm+ReLU emitter. Constructor signatures, attribute meaning, bias rules and
// error messages follow the reference's ROperator_Gemm<T> (src/SOFIE_core/inc/SOFIE/
// ROperator_Gemm.hxx:47-67,139-269,292-390); what is emitted is one call of sofie_hip_gemm_f32
// with the bias broadcast and the activation fused in the kernel epilogue, instead of
// std::copy(bias) + BLAS::sgemm_ + a scalar ReLU loop.
#ifndef SOFIE_ROPERATOR_GEMM
#define SOFIE_ROPERATOR_GEMM

#include <iomanip>
#include <limits>
#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

inline std::string FloatLiteral(float v)
{
   std::stringstream s;
   s << "static_cast<float>(" << std::setprecision(std::numeric_limits<float>::max_digits10) << v << ")";
   return s.str();
}

template <typename T>
class ROperator_Gemm final : public ROperator {
private:
   float fAttrAlpha = 1.0;
   float fAttrBeta = 1.0;
   int_t fAttrTransA = 0;
   int_t fAttrTransB = 0;
   std::string fNA, fNB, fNC = "", fNY;
   EActivationType fActivation = EActivationType::UNDEFINED;
   std::vector<size_t> fShapeA, fShapeB, fShapeC, fShapeY;
   int fBiasKind = 0;   // SOFIE_BIAS_*
   size_t fStack = 1;                       // stacked products (numpy.matmul on rank > 2 operands)
   std::vector<size_t> fStackA, fStackB;    // matrix index of A and B for every stacked product
   std::vector<size_t> fLeadY;              // leading dimensions of Y
   std::vector<size_t> fLeadStrideA, fLeadStrideB;   // element strides of A and B along them (0: broadcast)
   static constexpr size_t SOFIE_GEMM_MAX_LEAD_DIMS = 6;   // SOFIE_GEMM_MAX_LEAD of the kernel library

public:
   // One layer of a chain of fully connected layers (RModel::FuseGemmChain): y = act(x W + bias), W [K, N].
   struct ChainLayer {
      std::string weights, bias;   // initialized tensors; bias "" if there is none
      size_t K = 0, N = 0;
      bool relu = false;
   };
   static constexpr size_t kChainMaxLayers = 16;    // SOFIE_MLP_MAX_LAYERS of the kernel library
   static constexpr size_t kChainMaxWidth = 512;    // widths the emitter joins (the kernel takes up to SOFIE_MLP_MAX_WIDTH)

private:
   std::vector<ChainLayer> fChain;   // on the first operator of a chain: every layer, its own included

public:
   ROperator_Gemm() {}
   ROperator_Gemm(float alpha, float beta, int_t transA, int_t transB, std::string nameA, std::string nameB,
                  std::string nameY, EActivationType activation = EActivationType::UNDEFINED)
      : fAttrAlpha(alpha), fAttrBeta(beta), fAttrTransA(transA), fAttrTransB(transB), fNA(UTILITY::Clean_name(nameA)),
        fNB(UTILITY::Clean_name(nameB)), fNY(UTILITY::Clean_name(nameY)), fActivation(activation)
   {
      static_assert(std::is_same<T, float>::value, "TMVA::SOFIE - Unsupported type parsing a Gemm operator");
      fInputTensorNames = {fNA, fNB};
      fOutputTensorNames = {fNY};
   }
   ROperator_Gemm(float alpha, float beta, int_t transA, int_t transB, std::string nameA, std::string nameB,
                  std::string nameC, std::string nameY, EActivationType activation = EActivationType::UNDEFINED)
      : fAttrAlpha(alpha), fAttrBeta(beta), fAttrTransA(transA), fAttrTransB(transB), fNA(UTILITY::Clean_name(nameA)),
        fNB(UTILITY::Clean_name(nameB)), fNC(UTILITY::Clean_name(nameC)), fNY(UTILITY::Clean_name(nameY)),
        fActivation(activation)
   {
      static_assert(std::is_same<T, float>::value, "TMVA::SOFIE - Unsupported type parsing a Gemm operator");
      fInputTensorNames = {fNA, fNB, fNC};
      fOutputTensorNames = {fNY};
   }

   std::string Kind() const override { return "Gemm"; }
   bool FuseActivation(EActivationType act) override
   {
      if (act != EActivationType::RELU || fActivation != EActivationType::UNDEFINED) return false;
      fActivation = act;
      return true;
   }

   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return {input[0]}; }

   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      if (input.size() > 3) throw std::runtime_error("TMVA SOFIE Gemm Op Shape Inference only need 2 or 3 input tensor");
      for (auto &i : input)
         if (i.size() < 2)
            throw std::runtime_error("TMVA SOFIE Gemm Op Shape Inference only accept input tensor with >=2 dimensions");
      if (input.size() == 3) return {input[2]};   // with three inputs the shape of Y is the shape of C
      // the last two dimensions multiply; leading dimensions of stacked operands broadcast against each other
      // (reference :93-122, numpy.matmul)
      const size_t ra = input[0].size(), rb = input[1].size();
      std::vector<size_t> a(input[0].end() - 2, input[0].end()), b(input[1].end() - 2, input[1].end());
      if (fAttrTransA) std::reverse(a.begin(), a.end());
      if (fAttrTransB) std::reverse(b.begin(), b.end());
      std::vector<size_t> y;
      const size_t lead = std::max(ra, rb) - 2;
      for (size_t i = 0; i < lead; ++i) {
         const size_t da = i + ra >= lead + 2 ? input[0][i + ra - lead - 2] : 1;
         const size_t db = i + rb >= lead + 2 ? input[1][i + rb - lead - 2] : 1;
         if (da != db && da != 1 && db != 1)
            throw std::runtime_error("TMVA SOFIE Gemm Op - invalid input shapes " + std::to_string(da) + " and " +
                                     std::to_string(db));
         y.push_back(da == 1 ? db : da);
      }
      y.push_back(a[0]);
      y.push_back(b[1]);
      return {y};
   }

   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNA) || !model.CheckIfTensorAlreadyExist(fNB))
         throw std::runtime_error("TMVA SOFIE Gemm Op Input Tensor " + fNA + " or " + fNB + " is not found in model");
      if (fNC != "" && !model.CheckIfTensorAlreadyExist(fNC))
         throw std::runtime_error("TMVA SOFIE Gemm Op Input Tensor" + fNC + " is not found in model");
      fShapeA = model.GetTensorShape(fNA);
      fShapeB = model.GetTensorShape(fNB);
      // a rank-1 A gets a leading 1, a rank-1 B a trailing 1, removed again from Y (reference :158-177)
      bool prependOne = false, appendOne = false;
      if (fShapeA.size() == 1) { fShapeA.insert(fShapeA.begin(), 1); prependOne = true; }
      if (fShapeB.size() == 1) { fShapeB.push_back(1); appendOne = true; }
      // Stacked operands (rank > 2, numpy.matmul): the shorter shape gets leading ones (reference :180-187), the
      // leading dimensions broadcast, and the emitted code runs one product per stacked matrix. The reference
      // loops over the stack too (:353-387) but hands every iteration the first matrices of A and B; here each
      // product reads its own.
      std::vector<size_t> fullY = ShapeInference({fShapeA, fShapeB})[0];
      {
         const size_t rank = fullY.size();
         std::vector<size_t> la(fShapeA), lb(fShapeB);
         la.insert(la.begin(), rank - la.size(), 1);
         lb.insert(lb.begin(), rank - lb.size(), 1);
         fStack = 1;
         fStackA.clear();
         fStackB.clear();
         // element strides of A and B along every leading dimension (0 where the operand is broadcast)
         fLeadStrideA.assign(rank - 2, 0);
         fLeadStrideB.assign(rank - 2, 0);
         {
            size_t sa = la[rank - 2] * la[rank - 1], sb = lb[rank - 2] * lb[rank - 1];
            for (size_t i = rank - 2; i-- > 0;) {
               fLeadStrideA[i] = la[i] != 1 ? sa : 0;
               fLeadStrideB[i] = lb[i] != 1 ? sb : 0;
               sa *= la[i];
               sb *= lb[i];
            }
         }
         // offsets (in matrices) of A and B for every stacked product, row-major over the leading dimensions
         for (size_t i = 0; i + 2 < rank; ++i) fStack *= fullY[i];
         for (size_t idx = 0; idx < fStack; ++idx) {
            size_t rem = idx, oa = 0, ob = 0, sa = 1, sb = 1;
            for (size_t i = rank - 2; i-- > 0;) {
               const size_t pos = rem % fullY[i];
               rem /= fullY[i];
               if (la[i] != 1) oa += pos * sa;
               if (lb[i] != 1) ob += pos * sb;
               sa *= la[i];
               sb *= lb[i];
            }
            fStackA.push_back(oa);
            fStackB.push_back(ob);
         }
         fShapeA.assign(la.end() - 2, la.end());
         fShapeB.assign(lb.end() - 2, lb.end());
         fLeadY.assign(fullY.begin(), fullY.end() - 2);
      }
      std::vector<size_t> a = fShapeA, b = fShapeB;
      if (fAttrTransA) std::reverse(a.begin(), a.end());
      if (fAttrTransB) std::reverse(b.begin(), b.end());
      if (a[1] != b[0])
         throw std::runtime_error("TMVA SOFIE Gemm Op " + fNY + " has invalid shape" + ConvertShapeToString(fShapeA) + " x " +
                                  ConvertShapeToString(fShapeB));
      fShapeY = {a[0], b[1]};
      if (fStack > 1 && fNC != "")
         throw std::runtime_error("TMVA SOFIE Gemm Op " + fNY + ": a bias on stacked operands is not supported by the device emission");
      if (model.GetTensorType(fNA) != ETensorType::FLOAT || model.GetTensorType(fNB) != ETensorType::FLOAT)
         throw std::runtime_error("TMVA SOFIE Gemm Op " + fNY + ": only float tensors are supported");
      if (fNC != "") {
         fShapeC = model.GetTensorShape(fNC);
         const size_t lenC = ConvertShapeToLength(fShapeC), M = fShapeY[0], N = fShapeY[1];
         // unidirectional broadcast of C to [M,N] happens inside the kernel epilogue; the reference
         // materialises the broadcast tensor in the Session constructor (:271-290)
         if (lenC == M * N && (fShapeC.size() < 2 || fShapeC.back() == N)) fBiasKind = 2;      // full
         else if (lenC == N && fShapeC.back() == N) fBiasKind = 1;                              // one row
         else if (lenC == M && fShapeC.size() == 2 && fShapeC[1] == 1) fBiasKind = 3;           // one column
         else if (lenC == 1 && model.IsInitializedTensor(fNC)) {
            // scalar: expanded to one row at generation time
            float v = static_cast<float *>(model.GetInitializedTensorData(fNC).get())[0];
            std::shared_ptr<void> row(malloc(N * sizeof(float)), free);
            std::fill_n(static_cast<float *>(row.get()), N, v);
            model.UpdateInitializedTensor(fNC, ETensorType::FLOAT, {N}, row);
            fShapeC = {N};
            fBiasKind = 1;
         } else
            throw std::runtime_error("TMVA SOFIE Gemm Op " + fNY + " Bias tensor has not correct size " +
                                     ConvertShapeToString(fShapeC) + " output shape " + ConvertShapeToString(fShapeY));
      }
      std::vector<size_t> shapeY = fLeadY;
      shapeY.insert(shapeY.end(), fShapeY.begin(), fShapeY.end());
      if (prependOne) shapeY.erase(shapeY.end() - 2);
      if (appendOne) shapeY.pop_back();
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNA), shapeY);
      model.AddNeededStdLib("algorithm");
   }

   // --- chains of fully connected layers ----------------------------------------------------------------------
   // This operator can be a layer of a chain: a plain product of a [M, K] activation with a constant [K, N] (or
   // [N, K] with transB) matrix, alpha 1, a constant bias of one row added once (beta 1) or none, widths the
   // one-launch kernel is meant for.
   bool ChainCandidate(const RModel &model) const
   {
      if (fShapeY.empty() || fStack != 1 || fAttrTransA || fAttrAlpha != 1.0f) return false;
      if (!model.IsInitializedTensor(fNB)) return false;
      if (!fNC.empty() && (fBiasKind != 1 || fAttrBeta != 1.0f || !model.IsInitializedTensor(fNC))) return false;
      const size_t k = fShapeA[1], n = fShapeY[1];
      return k >= 1 && n >= 1 && k <= kChainMaxWidth && n <= kChainMaxWidth;
   }
   const std::string &NameA() const { return fNA; }
   const std::string &NameB() const { return fNB; }
   const std::string &NameY() const { return fNY; }
   bool TransB() const { return fAttrTransB != 0; }
   size_t Rows() const { return fShapeY[0]; }
   size_t MultiplyAdds() const { return fShapeA[1] * fShapeY[1]; }
   bool IsChainHead() const { return !fChain.empty(); }
   // The constant matrix as [K, N]: a transposed one is rewritten once, here, at generation time.
   void MakeWeightsKByN(RModel &model)
   {
      if (!fAttrTransB) return;
      const size_t n = fShapeB[0], k = fShapeB[1];
      const float *src = static_cast<const float *>(model.GetInitializedTensorData(fNB).get());
      std::shared_ptr<void> dst(malloc(n * k * sizeof(float)), free);
      float *d = static_cast<float *>(dst.get());
      for (size_t i = 0; i < n; ++i)
         for (size_t j = 0; j < k; ++j) d[j * n + i] = src[i * k + j];
      model.UpdateInitializedTensor(fNB, ETensorType::FLOAT, {k, n}, dst);
      fShapeB = {k, n};
      fAttrTransB = 0;
   }
   ChainLayer AsLayer() const
   {
      ChainLayer l;
      l.weights = fNB;
      l.bias = fNC;
      l.K = fShapeA[1];
      l.N = fShapeY[1];
      l.relu = fActivation == EActivationType::RELU;
      return l;
   }
   // This operator becomes the first layer of a chain that ends in the tensor `last` ([M, N of the last layer]):
   // it reads the weights and biases of every layer and writes `last` only.
   void BecomeChainHead(const std::vector<ChainLayer> &layers, const std::string &last)
   {
      fChain = layers;
      fOutputTensorNames = {last};
      fInputTensorNames = {fNA};
      for (auto &l : fChain) {
         fInputTensorNames.push_back(l.weights);
         if (!l.bias.empty()) fInputTensorNames.push_back(l.bias);
      }
   }

   // the rows of A are the batch: not with a transposed A, stacked operands or a bias of one value per row
   bool SetRuntimeBatch(const std::string &expr, size_t capacity) override
   {
      if (fAttrTransA || fStack > 1 || fBiasKind == 3) return false;
      return ROperator::SetRuntimeBatch(expr, capacity);
   }

   std::string Generate(std::string opName) override
   {
      opName = "op_" + opName;
      if (fShapeA.empty() || fShapeB.empty() || fShapeY.empty() || (fNC != "" && fShapeC.empty()))
         throw std::runtime_error("TMVA SOFIE Gemm Op called to Generate without being initialized first");
      if (fNC.empty() && fAttrBeta != 0)
         throw std::runtime_error("TMVA SOFIE Gemm Op " + opName + " Bias tensor is not present but beta value in Gemm is not zero");
      const size_t m = fShapeY[0], n = fShapeY[1];
      const size_t k = fAttrTransA ? fShapeA[0] : fShapeA[1];
      std::stringstream out;
      if (!fChain.empty()) {
         // every layer of the chain in one launch; the activations between the layers stay on chip
         out << "\n//--------- Gemm x " << fChain.size() << " (chain of fully connected layers)\n";
         out << SP << "{\n";
         out << SP << SP << "static const int " << opName << "_dims[] = {" << fChain.front().K;
         for (auto &l : fChain) out << ", " << l.N;
         out << "};\n";
         out << SP << SP << "const float *" << opName << "_w[] = {";
         for (size_t i = 0; i < fChain.size(); ++i) out << (i ? ", " : "") << "tensor_" << fChain[i].weights;
         out << "};\n";
         out << SP << SP << "const float *" << opName << "_b[] = {";
         for (size_t i = 0; i < fChain.size(); ++i)
            out << (i ? ", " : "") << (fChain[i].bias.empty() ? std::string("nullptr") : "tensor_" + fChain[i].bias);
         out << "};\n";
         out << SP << SP << "static const int " << opName << "_act[] = {";
         for (size_t i = 0; i < fChain.size(); ++i) out << (i ? ", " : "") << (fChain[i].relu ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE");
         out << "};\n";
         out << SP << SP << "Check(sofie_hip_mlp_f32(fCtx, " << fChain.size() << ", " << opName << "_dims, " << opName << "_w, "
             << opName << "_b, " << opName << "_act, tensor_" << fNA << ", " << fChain.front().K << ", tensor_"
             << fOutputTensorNames[0] << ", " << fChain.back().N << ", " << BatchCount(m) << "), \"Gemm chain " << opName << "\");\n";
         out << SP << "}\n";
         return out.str();
      }
      out << "\n//--------- Gemm\n";
      const std::string act = fActivation == EActivationType::RELU ? "SOFIE_ACT_RELU" : "SOFIE_ACT_NONE";
      if (fStack > 1) {
         // every product of the stack in one launch: the kernel finds its matrices of A and B from the position
         // along the leading dimensions (broadcast dimensions have stride 0)
         if (fLeadY.size() > SOFIE_GEMM_MAX_LEAD_DIMS)
            throw std::runtime_error("TMVA SOFIE Gemm Op " + fNY + ": more than " + std::to_string(SOFIE_GEMM_MAX_LEAD_DIMS) +
                                     " stacked dimensions are not supported by the device emission");
         out << SP << "{\n";
         out << SP << SP << "static const int " << opName << "_lead[] = {";
         for (size_t i = 0; i < fLeadY.size(); ++i) out << (i ? ", " : "") << fLeadY[i];
         out << "};\n";
         out << SP << SP << "static const long long " << opName << "_sa[] = {";
         for (size_t i = 0; i < fLeadY.size(); ++i) out << (i ? ", " : "") << fLeadStrideA[i];
         out << "};\n";
         out << SP << SP << "static const long long " << opName << "_sb[] = {";
         for (size_t i = 0; i < fLeadY.size(); ++i) out << (i ? ", " : "") << fLeadStrideB[i];
         out << "};\n";
         out << SP << SP << "Check(sofie_hip_gemm_f32_stacked(fCtx, " << (fAttrTransA ? 1 : 0) << ", " << (fAttrTransB ? 1 : 0) << ", " << m
             << ", " << n << ", " << k << ", " << FloatLiteral(fAttrAlpha) << ", tensor_" << fNA << ", " << fShapeA[1] << ", tensor_"
             << fNB << ", " << fShapeB[1] << ", tensor_" << fNY << ", " << n << ", " << fLeadY.size() << ", " << opName << "_lead, "
             << opName << "_sa, " << opName << "_sb, " << act << "), \"Gemm " << opName << "\");\n";
         out << SP << "}\n";
         return out.str();
      }
      out << SP << "Check(sofie_hip_gemm_f32(fCtx, " << (fAttrTransA ? 1 : 0) << ", " << (fAttrTransB ? 1 : 0) << ", " << BatchCount(m) << ", "
          << n << ", " << k << ", " << FloatLiteral(fAttrAlpha) << ", tensor_" << fNA << ", " << fShapeA[1] << ", tensor_" << fNB
          << ", " << fShapeB[1] << ", " << FloatLiteral(fNC.empty() ? 0.0f : fAttrBeta) << ", "
          << (fNC.empty() ? std::string("nullptr") : "tensor_" + fNC) << ", " << fBiasKind << ", tensor_" << fNY << ", " << n << ", "
          << act << "), \"Gemm " << opName << "\");\n";
      return out.str();
   }

   // Host form, as the reference emits it (ROperator_Gemm.hxx:292-390): the bias broadcast to [M,N] is copied into Y,
   // then one BLAS::sgemm_ in the column-major reading of the row-major tensors (Y^T = op(B)^T op(A)^T, so B comes
   // first and the leading dimension of Y is N), then the ReLU loop. Stacked operands run one such product per
   // matrix, each on its own matrices of A and B.
   std::string GenerateHost(std::string opName) override
   {
      opName = "op_" + opName;
      if (fShapeA.empty() || fShapeB.empty() || fShapeY.empty() || (fNC != "" && fShapeC.empty()))
         throw std::runtime_error("TMVA SOFIE Gemm Op called to Generate without being initialized first");
      if (fNC.empty() && fAttrBeta != 0)
         throw std::runtime_error("TMVA SOFIE Gemm Op " + opName + " Bias tensor is not present but beta value in Gemm is not zero");
      const size_t m = fShapeY[0], n = fShapeY[1];
      const size_t k = fAttrTransA ? fShapeA[0] : fShapeA[1];
      std::stringstream out;
      out << "\n//--------- Gemm\n";
      out << SP << "{\n";
      out << SP << SP << "char " << opName << "_transA = '" << (fAttrTransA ? "t" : "n") << "';\n";
      out << SP << SP << "char " << opName << "_transB = '" << (fAttrTransB ? "t" : "n") << "';\n";
      out << SP << SP << "int " << opName << "_m = " << BatchCount(m) << ";\n";
      out << SP << SP << "int " << opName << "_n = " << n << ";\n";
      out << SP << SP << "int " << opName << "_k = " << k << ";\n";
      out << SP << SP << "float " << opName << "_alpha = " << FloatLiteral(fAttrAlpha) << ";\n";
      out << SP << SP << "float " << opName << "_beta = " << FloatLiteral(fNC.empty() ? 0.0f : fAttrBeta) << ";\n";
      out << SP << SP << "int " << opName << "_lda = " << fShapeA[1] << ";\n";
      out << SP << SP << "int " << opName << "_ldb = " << fShapeB[1] << ";\n";
      if (!fNC.empty()) {
         const std::string rows = opName + "_m";
         if (fBiasKind == 2)
            out << SP << SP << "std::copy(tensor_" << fNC << ", tensor_" << fNC << " + static_cast<size_t>(" << rows << ") * " << n
                << ", tensor_" << fNY << ");\n";
         else if (fBiasKind == 1)
            out << SP << SP << "for (int row = 0; row < " << rows << "; ++row) std::copy(tensor_" << fNC << ", tensor_" << fNC << " + "
                << n << ", tensor_" << fNY << " + static_cast<size_t>(row) * " << n << ");\n";
         else
            out << SP << SP << "for (int row = 0; row < " << rows << "; ++row) std::fill_n(tensor_" << fNY
                << " + static_cast<size_t>(row) * " << n << ", " << n << ", tensor_" << fNC << "[row]);\n";
      }
      if (fStack > 1) {
         const size_t sizeA = fShapeA[0] * fShapeA[1], sizeB = fShapeB[0] * fShapeB[1];
         out << SP << SP << "static const size_t " << opName << "_offA[] = {";
         for (size_t i = 0; i < fStack; ++i) out << (i ? ", " : "") << fStackA[i] * sizeA;
         out << "};\n";
         out << SP << SP << "static const size_t " << opName << "_offB[] = {";
         for (size_t i = 0; i < fStack; ++i) out << (i ? ", " : "") << fStackB[i] * sizeB;
         out << "};\n";
         out << SP << SP << "for (size_t stack = 0; stack < " << fStack << "; ++stack)\n";
         out << SP << SP << SP << "BLAS::sgemm_(&" << opName << "_transB, &" << opName << "_transA, &" << opName << "_n, &" << opName
             << "_m, &" << opName << "_k, &" << opName << "_alpha, tensor_" << fNB << " + " << opName << "_offB[stack], &" << opName
             << "_ldb, tensor_" << fNA << " + " << opName << "_offA[stack], &" << opName << "_lda, &" << opName << "_beta, tensor_"
             << fNY << " + stack * " << m * n << ", &" << opName << "_n);\n";
      } else {
         out << SP << SP << "BLAS::sgemm_(&" << opName << "_transB, &" << opName << "_transA, &" << opName << "_n, &" << opName
             << "_m, &" << opName << "_k, &" << opName << "_alpha, tensor_" << fNB << ", &" << opName << "_ldb, tensor_" << fNA
             << ", &" << opName << "_lda, &" << opName << "_beta, tensor_" << fNY << ", &" << opName << "_n);\n";
      }
      if (fActivation == EActivationType::RELU) {
         out << SP << SP << "for (size_t id = 0; id < static_cast<size_t>(" << opName << "_m) * " << n * fStack << "; id++)\n";
         out << SP << SP << SP << "tensor_" << fNY << "[id] = ((tensor_" << fNY << "[id] > 0 )? tensor_" << fNY << "[id] : 0);\n";
      }
      out << SP << "}\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
