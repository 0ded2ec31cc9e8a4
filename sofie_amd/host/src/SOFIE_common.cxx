#include "SOFIE/SOFIE_common.hxx"

#include <cctype>

namespace SOFIE {

size_t GetTypeSize(ETensorType type)
{
   switch (type) {
   case ETensorType::FLOAT: return 4;
   case ETensorType::DOUBLE: return 8;
   case ETensorType::UINT8: return 1;
   case ETensorType::INT8: return 1;
   case ETensorType::FLOAT8E4M3FN: return 1;
   case ETensorType::UINT16: return 2;
   case ETensorType::INT16: return 2;
   case ETensorType::BFLOAT16: return 2;
   case ETensorType::FLOAT16: return 2;
   case ETensorType::INT32: return 4;
   case ETensorType::INT64: return 8;
   case ETensorType::UINT32: return 4;
   case ETensorType::UINT64: return 8;
   case ETensorType::BOOL: return 1;
   default: return 0;
   }
}

std::string ConvertTypeToString(ETensorType type)
{
   switch (type) {
   case ETensorType::FLOAT: return "float";
   case ETensorType::INT8: return "int8_t";
   case ETensorType::UINT8: return "uint8_t";
   case ETensorType::FLOAT8E4M3FN: return "uint8_t";    // storage type of an e4m3 code
   case ETensorType::BFLOAT16: return "uint16_t";       // storage type of a bf16 bit pattern
   case ETensorType::INT16: return "int16_t";
   case ETensorType::INT32: return "int32_t";
   case ETensorType::INT64: return "int64_t";
   case ETensorType::UINT16: return "uint16_t";
   case ETensorType::UINT32: return "uint32_t";
   case ETensorType::UINT64: return "uint64_t";
   case ETensorType::DOUBLE: return "double";
   case ETensorType::BOOL: return "bool";
   default: return "other_" + std::to_string((int)type);
   }
}

ETensorType ConvertStringToType(std::string type)
{
   if (type == "float32" || type == "float" || type == "Float") return ETensorType::FLOAT;
   if (type == "int64" || type == "int64_t") return ETensorType::INT64;
   if (type == "int32" || type == "int32_t") return ETensorType::INT32;
   if (type == "int8" || type == "int8_t") return ETensorType::INT8;
   if (type == "uint8" || type == "uint8_t") return ETensorType::UINT8;
   if (type == "double" || type == "float64") return ETensorType::DOUBLE;
   if (type == "bool") return ETensorType::BOOL;
   return ETensorType::UNDEFINED;
}

std::vector<Dim> ConvertShapeToDim(std::vector<size_t> shape)
{
   std::vector<Dim> ret(shape.size());
   for (size_t i = 0; i < shape.size(); i++) ret[i].dim = shape[i];
   return ret;
}

std::vector<size_t> ConvertShapeToInt(std::vector<Dim> shape)
{
   std::vector<size_t> ret(shape.size());
   for (size_t i = 0; i < shape.size(); i++) {
      if (!shape[i].isParam) {
         ret[i] = shape[i].dim;
         continue;
      }
      // a parameter that spells a non-negative number still counts as a fixed dimension
      char *end = nullptr;
      long v = std::strtol(shape[i].param.c_str(), &end, 10);
      if (shape[i].param.empty() || *end != '\0' || v < 0) return {};
      ret[i] = static_cast<size_t>(v);
   }
   return ret;
}

std::size_t ConvertShapeToLength(std::vector<size_t> shape)
{
   std::size_t len = 1;   // an empty shape is a scalar
   for (auto &d : shape) len *= d;
   return len;
}

std::string ConvertShapeToString(std::vector<size_t> shape)
{
   std::stringstream out;
   out << "{ ";
   for (size_t i = 0; i < shape.size(); i++) out << shape[i] << (i + 1 < shape.size() ? " , " : "");
   out << " }";
   return out.str();
}

std::string ConvertDynamicShapeToString(std::vector<Dim> shape)
{
   std::stringstream out;
   out << "{ ";
   for (size_t i = 0; i < shape.size(); i++) out << shape[i].GetVal() << (i + 1 < shape.size() ? " , " : "");
   out << " }";
   return out.str();
}

bool UTILITY::AreSameShape(const std::vector<size_t> &a, const std::vector<size_t> &b) { return a == b; }

std::string UTILITY::Clean_name(std::string s)
{
   std::replace(s.begin(), s.end(), '-', '_');
   s.erase(std::remove_if(s.begin(), s.end(), [](unsigned char c) { return !std::isalnum(c) && c != '_'; }), s.end());
   return s;
}

std::vector<size_t> UTILITY::ComputeStrideFromShape(const std::vector<size_t> &shape)
{
   std::vector<size_t> strides(shape.size(), 1);
   for (size_t i = shape.size(); i-- > 1;) strides[i - 1] = strides[i] * shape[i];
   return strides;
}

}   // namespace SOFIE
