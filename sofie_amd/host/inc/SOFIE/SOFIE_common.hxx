// Types and helpers shared by the graph IR (RModel) and the operator emitters.
// Mirrors the vocabulary of the reference's src/SOFIE_core/inc/SOFIE/SOFIE_common.hxx
// (ETensorType, EActivationType, Dim, TensorInfo, InitializedTensor, UTILITY::Clean_name,
// ConvertShapeTo*), without any ROOT dependency, and extends the type table to the element
// types the quantized operators need (the reference maps int8/uint8 to "other_<n>",
// src/SOFIE_core/src/SOFIE_common.cxx:56-89).
#ifndef SOFIE_SOFIE_COMMON
#define SOFIE_SOFIE_COMMON

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

namespace SOFIE {

// numeric values follow ONNX TensorProto.DataType, as in the reference (:29-32)
enum class ETensorType {
   UNDEFINED = 0, FLOAT = 1, UINT8 = 2, INT8 = 3, UINT16 = 4, INT16 = 5, INT32 = 6, INT64 = 7, STRING = 8,
   BOOL = 9, FLOAT16 = 10, DOUBLE = 11, UINT32 = 12, UINT64 = 13, COMPLEX64 = 14, COMPLEX28 = 15,
   BFLOAT16 = 16, FLOAT8E4M3FN = 17
};

enum class EActivationType { UNDEFINED = 0, RELU = 1, SOFTMAX = 2, SIGMOID = 3, LEAKYRELU = 4, TANH = 5, ELU = 6 };

typedef std::int64_t int_t;

size_t GetTypeSize(ETensorType type);
// C++ spelling of the element type in generated code ("float", "int8_t", ...)
std::string ConvertTypeToString(ETensorType type);
ETensorType ConvertStringToType(std::string type);

struct Dim {
   bool isParam = false;
   size_t dim = 0;
   std::string param;
   Dim() {}
   Dim(const std::string &p, size_t d = 0) : isParam(true), dim(d), param(p) {}
   Dim(size_t d) : dim(d) {}
   std::string GetVal() const { return isParam ? param : std::to_string(dim); }
};

struct TensorInfo {
   ETensorType type;
   std::vector<size_t> shape;
};

class InitializedTensor {
public:
   InitializedTensor() = default;
   InitializedTensor(ETensorType type, const std::vector<size_t> &shape, std::shared_ptr<void> data)
      : fType(type), fShape(shape), fData(data) {}
   ETensorType const &type() const { return fType; }
   std::vector<size_t> const &shape() const { return fShape; }
   std::shared_ptr<void> const &sharedptr() const { return fData; }
   template <class T> T const *data() const { return static_cast<T const *>(fData.get()); }
   bool IsWeightTensor() const { return fWritable; }
   void SetNotWritable() { fWritable = false; }
private:
   ETensorType fType = ETensorType::UNDEFINED;
   std::vector<size_t> fShape;
   std::shared_ptr<void> fData;
   bool fWritable = true;   // written to / read from the weight file
};

template <typename T> ETensorType GetTemplatedType(T /*obj*/)
{
   if (std::is_same<T, float>::value) return ETensorType::FLOAT;
   if (std::is_same<T, uint8_t>::value) return ETensorType::UINT8;
   if (std::is_same<T, int8_t>::value) return ETensorType::INT8;
   if (std::is_same<T, uint16_t>::value) return ETensorType::UINT16;
   if (std::is_same<T, int16_t>::value) return ETensorType::INT16;
   if (std::is_same<T, int32_t>::value) return ETensorType::INT32;
   if (std::is_same<T, int64_t>::value) return ETensorType::INT64;
   if (std::is_same<T, bool>::value) return ETensorType::BOOL;
   if (std::is_same<T, double>::value) return ETensorType::DOUBLE;
   if (std::is_same<T, uint32_t>::value) return ETensorType::UINT32;
   if (std::is_same<T, uint64_t>::value) return ETensorType::UINT64;
   return ETensorType::UNDEFINED;
}

std::vector<Dim> ConvertShapeToDim(std::vector<size_t> shape);
std::vector<size_t> ConvertShapeToInt(std::vector<Dim> shape);
std::size_t ConvertShapeToLength(std::vector<size_t> shape);
std::string ConvertShapeToString(std::vector<size_t> shape);
std::string ConvertDynamicShapeToString(std::vector<Dim> shape);

namespace UTILITY {
bool AreSameShape(const std::vector<size_t> &, const std::vector<size_t> &);
// keeps [A-Za-z0-9_], turns '-' into '_' (reference: SOFIE_common.cxx:394-400)
std::string Clean_name(std::string input_tensor_name);
// row-major element strides of a dense tensor (reference: SOFIE_common.cxx:402-413)
std::vector<size_t> ComputeStrideFromShape(const std::vector<size_t> &shape);
}   // namespace UTILITY

}   // namespace SOFIE
#endif
