// Einsum emitter. Constructor, equation syntax, label bookkeeping and error messages follow the reference's
// ROperator_Einsum<T> (src/SOFIE_core/inc/SOFIE/ROperator_Einsum.hxx:40-112,124-200):
//   - the equation needs an explicit "->"; labels are single alphanumeric characters, blanks are ignored;
//   - the output shape comes from the label sizes; labels missing from the output are summed, in the order
//     of a std::map<char,...> (sorted by character), the first one as the outermost loop;
//   - two operands with one summed label that sits in the last two positions of both are a (stacked)
//     matrix product ("nn", "tn", "nt", "tt", :181-197).
// Emitted code: the matrix-product case is one sofie_hip_gemm_f32 call per stacked matrix where the reference
// emits BLAS::sgemm_ inside loops over the leading output labels (:280-336); every other equation is one
// sofie_hip_einsum_f32 call where the reference emits a nest of host loops (:236-278).
// Checked here, and not by the reference: that a label has the same size wherever it appears, that the rank
// of an operand equals its number of labels, and that the two free labels of a matrix product are the last two
// output labels in this order (otherwise the equation takes the general path instead of a wrong product).
#ifndef SOFIE_ROPERATOR_EINSUM
#define SOFIE_ROPERATOR_EINSUM

#include <algorithm>
#include <cctype>
#include <iostream>
#include <map>
#include <sstream>

#include "SOFIE/RModel.hxx"
#include "SOFIE/ROperator.hxx"

namespace SOFIE {

template <typename T>
class ROperator_Einsum final : public ROperator {
private:
   std::vector<std::string> fNInputs;
   std::string fNY;
   std::vector<std::string> fInputLabels;
   std::string fOutputLabels;
   std::string fSumLabels;
   std::string fGemmType;
   std::vector<int> fSumDims;
   std::vector<std::vector<size_t>> fShapeInputs;
   std::vector<size_t> fShapeY;
   std::map<char, size_t> fExtent;
   bool fInitialized = false;

   static bool CheckLabels(const std::string &labels)
   {
      for (char c : labels)
         if (!std::isalnum(static_cast<unsigned char>(c))) {
            std::cout << "Wrong tensor label " << labels << std::endl;
            return false;
         }
      return true;   // no label at all is a scalar
   }

   // element stride of every label of `all` in an operand with these labels and this shape
   static std::vector<long long> LabelStrides(const std::string &all, const std::string &labels, const std::vector<size_t> &shape)
   {
      const auto strides = UTILITY::ComputeStrideFromShape(shape);
      std::vector<long long> r(all.size(), 0);
      for (size_t j = 0; j < labels.size(); ++j) r[all.find(labels[j])] += (long long)strides[j];
      return r;
   }

public:
   ROperator_Einsum() {}
   ROperator_Einsum(const std::string &equation, const std::vector<std::string> &namesX, const std::string &nameY)
      : fNInputs(namesX.size()), fNY(UTILITY::Clean_name(nameY))
   {
      if (!std::is_same<T, float>::value)
         throw std::runtime_error("TMVA SOFIE Encountered unsupported type parsing an Einsum operator");
      for (size_t i = 0; i < namesX.size(); i++) fNInputs[i] = UTILITY::Clean_name(namesX[i]);
      if (!ParseEquation(equation))
         throw std::runtime_error("TMVA SOFIE Einsum Op: Error parsing the equation " + equation);
      fInputTensorNames = fNInputs;
      fOutputTensorNames = {fNY};
   }

   std::string Kind() const override { return "Einsum"; }
   // no label is known to be the batch
   bool SetRuntimeBatch(const std::string &, size_t) override { return false; }
   const std::string &GemmType() const { return fGemmType; }

   bool ParseEquation(const std::string &input_equation)
   {
      std::string eq(input_equation);
      eq.erase(std::remove(eq.begin(), eq.end(), ' '), eq.end());
      const size_t arrow = eq.find("->");
      if (arrow == std::string::npos) {
         std::cout << "'->' not found in the equation." << std::endl;
         return false;
      }
      const std::string in = eq.substr(0, arrow);
      fOutputLabels = eq.substr(arrow + 2);
      fInputLabels.clear();
      size_t start = 0;
      for (size_t comma; (comma = in.find(',', start)) != std::string::npos; start = comma + 1)
         fInputLabels.push_back(in.substr(start, comma - start));
      fInputLabels.push_back(in.substr(start));
      for (auto &l : fInputLabels)
         if (!CheckLabels(l)) return false;
      if (!CheckLabels(fOutputLabels)) {
         std::cout << "invalid output label" << std::endl;
         return false;
      }
      if (fInputLabels.size() != fNInputs.size()) {
         std::cout << "Invalid number of input labels found " << fInputLabels.size() << " for #inputs = " << fNInputs.size()
                   << std::endl;
         return false;
      }
      return true;
   }

   std::vector<ETensorType> TypeInference(std::vector<ETensorType> input) override { return {input[0]}; }

   std::vector<std::vector<size_t>> ShapeInference(std::vector<std::vector<size_t>> input) override
   {
      std::map<char, size_t> extent;
      for (size_t i = 0; i < input.size() && i < fInputLabels.size(); ++i)
         for (size_t j = 0; j < input[i].size() && j < fInputLabels[i].size(); ++j) extent[fInputLabels[i][j]] = input[i][j];
      std::vector<size_t> y;
      for (char l : fOutputLabels) y.push_back(extent.count(l) ? extent[l] : 0);
      return {y};
   }

   void Initialize(RModel &model) override
   {
      fShapeInputs.clear();
      fExtent.clear();
      for (size_t i = 0; i < fNInputs.size(); ++i) {
         const std::string &name = fNInputs[i];
         if (!model.CheckIfTensorAlreadyExist(name))
            throw std::runtime_error(std::string("TMVA SOFIE Einsum Op Input Tensor ") + name + "is not found in model");
         if (model.GetTensorType(name) != ETensorType::FLOAT)
            throw std::runtime_error("TMVA SOFIE Einsum Op: only float tensors are supported, " + name + " is not");
         const auto shape = model.GetTensorShape(name);
         const std::string &labels = fInputLabels[i];
         if (shape.size() != labels.size())
            throw std::runtime_error(std::string("TMVA SOFIE Einsum Op Input Tensor has invalid label or shape ") + labels + " " +
                                     ConvertShapeToString(shape));
         for (size_t j = 0; j < shape.size(); ++j) {
            auto known = fExtent.find(labels[j]);
            if (known != fExtent.end() && known->second != shape[j])
               throw std::runtime_error(std::string("TMVA SOFIE Einsum Op : label ") + labels[j] + " has two sizes, " +
                                        std::to_string(known->second) + " and " + std::to_string(shape[j]));
            fExtent[labels[j]] = shape[j];
         }
         fShapeInputs.push_back(shape);
      }
      fShapeY.clear();
      for (size_t j = 0; j < fOutputLabels.size(); ++j) {
         const char l = fOutputLabels[j];
         if (fExtent.count(l) == 0)
            throw std::runtime_error(std::string("TMVA SOFIE Einsum Op : output label ") + std::string(1, l) + " is not present in inputs");
         if (fOutputLabels.find(l) != j)
            throw std::runtime_error(std::string("TMVA SOFIE Einsum Op : output label ") + std::string(1, l) + " appears twice");
         fShapeY.push_back(fExtent[l]);
      }
      fSumLabels = "";
      fSumDims.clear();
      for (auto &l : fExtent)
         if (fOutputLabels.find(l.first) == std::string::npos) {
            fSumLabels += l.first;
            fSumDims.push_back((int)l.second);
         }
      fGemmType = MatrixProductType();
      if (fGemmType.empty()) {
         if (fNInputs.size() > 4 || fOutputLabels.size() + fSumLabels.size() > 12)
            throw std::runtime_error("TMVA SOFIE Einsum Op : at most 4 operands and 12 distinct labels are supported by the device emission");
      }
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNInputs[0]), fShapeY);
      if (model.Verbose()) {
         std::cout << "Einsum op ";
         for (size_t i = 0; i < fNInputs.size(); i++)
            std::cout << (i ? ", " : "") << fNInputs[i] << " " << ConvertShapeToString(fShapeInputs[i]) << " " << fInputLabels[i];
         std::cout << " --> " << fNY << "  " << ConvertShapeToString(fShapeY) << "  " << fOutputLabels
                   << (fGemmType.empty() ? "" : "  as matrix product " + fGemmType) << std::endl;
      }
      fInitialized = true;
   }

   // "nn" / "tn" / "nt" / "tt" when the equation is a stacked matrix product, "" otherwise
   std::string MatrixProductType() const
   {
      if (fNInputs.size() != 2 || fSumLabels.size() != 1) return "";
      const std::string &la = fInputLabels[0], &lb = fInputLabels[1], &ly = fOutputLabels;
      if (la.size() < 2 || lb.size() < 2 || ly.size() < 2) return "";
      auto distinct = [](const std::string &s) {
         for (size_t i = 0; i < s.size(); ++i)
            if (s.find(s[i]) != i) return false;
         return true;
      };
      if (!distinct(la) || !distinct(lb)) return "";
      const char s = fSumLabels[0];
      const size_t pa = la.find(s), pb = lb.find(s);
      if (pa == std::string::npos || pb == std::string::npos || pa + 2 < la.size() || pb + 2 < lb.size()) return "";
      const bool ta = pa == la.size() - 2, tb = pb == lb.size() - 1;
      const char m = ta ? la.back() : la[la.size() - 2];
      const char n = tb ? lb[lb.size() - 2] : lb.back();
      // the free labels are the rows and columns of y, in this order, and belong to one operand each
      if (m == n || ly[ly.size() - 2] != m || ly.back() != n) return "";
      if (lb.find(m) != std::string::npos || la.find(n) != std::string::npos) return "";
      // every leading label of an operand numbers the stacked matrices of y
      const std::string lead = ly.substr(0, ly.size() - 2);
      for (size_t i = 0; i + 2 < la.size(); ++i)
         if (lead.find(la[i]) == std::string::npos) return "";
      for (size_t i = 0; i + 2 < lb.size(); ++i)
         if (lead.find(lb[i]) == std::string::npos) return "";
      return std::string(ta ? "t" : "n") + (tb ? "t" : "n");
   }

   std::string Generate(std::string opName) override
   {
      opName = "op_" + opName;
      if (!fInitialized || fShapeY.size() != fOutputLabels.length())
         throw std::runtime_error("TMVA SOFIE Einsum Op called to Generate without being initialized first");
      std::stringstream out;
      out << "\n//-------- Einsum   \n";
      if (!fGemmType.empty()) {
         out << SP << "// implementing Einsum using MatMul   \n";
         const auto &sa = fShapeInputs[0], &sb = fShapeInputs[1];
         const bool ta = fGemmType[0] == 't', tb = fGemmType[1] == 't';
         const size_t m = ta ? sa.back() : sa[sa.size() - 2];
         const size_t k = ta ? sa[sa.size() - 2] : sa.back();
         const size_t n = tb ? sb[sb.size() - 2] : sb.back();
         // offsets of the stacked matrices: y's leading labels in row-major order, each operand by its own strides
         const std::string lead = fOutputLabels.substr(0, fOutputLabels.size() - 2);
         const auto stA = LabelStrides(lead, fInputLabels[0].substr(0, fInputLabels[0].size() - 2),
                                       std::vector<size_t>(sa.begin(), sa.end() - 2));
         const auto stB = LabelStrides(lead, fInputLabels[1].substr(0, fInputLabels[1].size() - 2),
                                       std::vector<size_t>(sb.begin(), sb.end() - 2));
         size_t stack = 1;
         for (size_t i = 0; i + 2 < fShapeY.size(); ++i) stack *= fShapeY[i];
         std::vector<size_t> offA(stack, 0), offB(stack, 0);
         for (size_t idx = 0; idx < stack; ++idx) {
            size_t rem = idx;
            for (size_t i = lead.size(); i-- > 0;) {
               const size_t pos = rem % fShapeY[i];
               rem /= fShapeY[i];
               offA[idx] += pos * (size_t)stA[i] * sa[sa.size() - 2] * sa.back();
               offB[idx] += pos * (size_t)stB[i] * sb[sb.size() - 2] * sb.back();
            }
         }
         std::string pa, pb, py, indent = SP;
         if (stack > 1) {
            out << SP << "{\n";
            out << SP << SP << "static const size_t " << opName << "_a[] = {";
            for (size_t i = 0; i < stack; ++i) out << (i ? ", " : "") << offA[i];
            out << "};\n";
            out << SP << SP << "static const size_t " << opName << "_b[] = {";
            for (size_t i = 0; i < stack; ++i) out << (i ? ", " : "") << offB[i];
            out << "};\n";
            out << SP << SP << "for (size_t i = 0; i < " << stack << "; i++)\n";
            pa = " + " + opName + "_a[i]";
            pb = " + " + opName + "_b[i]";
            py = " + i * " + std::to_string(m * n);
            indent = SP + SP + SP;
         }
         out << indent << "Check(sofie_hip_gemm_f32(fCtx, " << (ta ? 1 : 0) << ", " << (tb ? 1 : 0) << ", " << m << ", " << n << ", " << k
             << ", 1.0f, tensor_" << fNInputs[0] << pa << ", " << sa.back() << ", tensor_" << fNInputs[1] << pb << ", " << sb.back()
             << ", 0.0f, nullptr, SOFIE_BIAS_NONE, tensor_" << fNY << py << ", " << n << ", SOFIE_ACT_NONE), \"Einsum " << opName
             << "\");\n";
         if (stack > 1) out << SP << "}\n";
         return out.str();
      }
      // general case: output labels first, then the summed labels in the reference's loop order
      const std::string all = fOutputLabels + fSumLabels;
      out << SP << "{\n";
      out << SP << SP << "static const int " << opName << "_extent[] = {";
      for (size_t l = 0; l < all.size(); ++l) out << (l ? ", " : "") << fExtent.at(all[l]);
      out << (all.empty() ? "1" : "") << "};\n";
      out << SP << SP << "static const long long " << opName << "_stride[] = {";
      bool first = true;
      for (size_t i = 0; i < fNInputs.size(); ++i)
         for (long long s : LabelStrides(all, fInputLabels[i], fShapeInputs[i])) {
            out << (first ? "" : ", ") << s;
            first = false;
         }
      out << (first ? "0" : "") << "};\n";
      out << SP << SP << "const float * " << opName << "_x[] = {";
      for (size_t i = 0; i < fNInputs.size(); ++i) out << (i ? ", " : "") << "tensor_" << fNInputs[i];
      out << "};\n";
      out << SP << SP << "Check(sofie_hip_einsum_f32(fCtx, " << fNInputs.size() << ", " << opName << "_x, " << all.size() << ", "
          << fOutputLabels.size() << ", " << opName << "_extent, " << opName << "_stride, tensor_" << fNY << "), \"Einsum " << opName
          << "\");\n";
      out << SP << "}\n";
      return out.str();
   }

   // Host form (reference ROperator_Einsum.hxx Generate): a product of two operands whose labels make it a (stacked)
   // matrix product is one BLAS::sgemm_ per stacked matrix; every other equation is the nest of loops over the output
   // labels and, inside, over the summed labels, written once as a helper that walks the labels like an odometer.
   std::string GenerateHost(std::string opName) override
   {
      opName = "op_" + opName;
      if (!fInitialized || fShapeY.size() != fOutputLabels.length())
         throw std::runtime_error("TMVA SOFIE Einsum Op called to Generate without being initialized first");
      std::stringstream out;
      out << "\n//-------- Einsum   \n";
      out << SP << "{\n";
      if (!fGemmType.empty()) {
         const auto &sa = fShapeInputs[0], &sb = fShapeInputs[1];
         const bool ta = fGemmType[0] == 't', tb = fGemmType[1] == 't';
         const size_t m = ta ? sa.back() : sa[sa.size() - 2];
         const size_t k = ta ? sa[sa.size() - 2] : sa.back();
         const size_t n = tb ? sb[sb.size() - 2] : sb.back();
         const std::string lead = fOutputLabels.substr(0, fOutputLabels.size() - 2);
         const auto stA = LabelStrides(lead, fInputLabels[0].substr(0, fInputLabels[0].size() - 2),
                                       std::vector<size_t>(sa.begin(), sa.end() - 2));
         const auto stB = LabelStrides(lead, fInputLabels[1].substr(0, fInputLabels[1].size() - 2),
                                       std::vector<size_t>(sb.begin(), sb.end() - 2));
         size_t stack = 1;
         for (size_t i = 0; i + 2 < fShapeY.size(); ++i) stack *= fShapeY[i];
         out << SP << SP << "static const size_t " << opName << "_a[] = {";
         for (size_t idx = 0; idx < stack; ++idx) {
            size_t rem = idx, oa = 0;
            for (size_t i = lead.size(); i-- > 0;) {
               oa += (rem % fShapeY[i]) * (size_t)stA[i] * sa[sa.size() - 2] * sa.back();
               rem /= fShapeY[i];
            }
            out << (idx ? ", " : "") << oa;
         }
         out << "};\n";
         out << SP << SP << "static const size_t " << opName << "_b[] = {";
         for (size_t idx = 0; idx < stack; ++idx) {
            size_t rem = idx, ob = 0;
            for (size_t i = lead.size(); i-- > 0;) {
               ob += (rem % fShapeY[i]) * (size_t)stB[i] * sb[sb.size() - 2] * sb.back();
               rem /= fShapeY[i];
            }
            out << (idx ? ", " : "") << ob;
         }
         out << "};\n";
         out << SP << SP << "char " << opName << "_transA = '" << (ta ? "t" : "n") << "', " << opName << "_transB = '" << (tb ? "t" : "n") << "';\n";
         out << SP << SP << "int " << opName << "_m = " << m << ", " << opName << "_n = " << n << ", " << opName << "_k = " << k << ", " << opName
             << "_lda = " << sa.back() << ", " << opName << "_ldb = " << sb.back() << ";\n";
         out << SP << SP << "float " << opName << "_alpha = 1.0, " << opName << "_beta = 0.0;\n";
         out << SP << SP << "for (size_t i = 0; i < " << stack << "; i++)\n";
         out << SP << SP << SP << "BLAS::sgemm_(&" << opName << "_transB, &" << opName << "_transA, &" << opName << "_n, &" << opName << "_m, &"
             << opName << "_k, &" << opName << "_alpha, tensor_" << fNInputs[1] << " + " << opName << "_b[i], &" << opName << "_ldb, tensor_"
             << fNInputs[0] << " + " << opName << "_a[i], &" << opName << "_lda, &" << opName << "_beta, tensor_" << fNY << " + i * " << m * n
             << ", &" << opName << "_n);\n";
         out << SP << "}\n";
         return out.str();
      }
      const std::string all = fOutputLabels + fSumLabels;
      out << SP << SP << "static const int " << opName << "_extent[] = {";
      for (size_t l = 0; l < all.size(); ++l) out << (l ? ", " : "") << fExtent.at(all[l]);
      out << (all.empty() ? "1" : "") << "};\n";
      out << SP << SP << "static const long long " << opName << "_stride[] = {";
      bool first = true;
      for (size_t i = 0; i < fNInputs.size(); ++i)
         for (long long s : LabelStrides(all, fInputLabels[i], fShapeInputs[i])) {
            out << (first ? "" : ", ") << s;
            first = false;
         }
      out << (first ? "0" : "") << "};\n";
      out << SP << SP << "const float * " << opName << "_x[] = {";
      for (size_t i = 0; i < fNInputs.size(); ++i) out << (i ? ", " : "") << "tensor_" << fNInputs[i];
      out << "};\n";
      out << SP << SP << "EinsumLoops(" << fNInputs.size() << ", " << opName << "_x, " << all.size() << ", " << fOutputLabels.size() << ", "
          << opName << "_extent, " << opName << "_stride, tensor_" << fNY << ");\n";
      out << SP << "}\n";
      return out.str();
   }
};

}   // namespace SOFIE
#endif
