// Every operator emitter of this build (the reference's OperatorList.hxx lists all of its own).
#include "SOFIE/ROperator_BatchNormalization.hxx"
#include "SOFIE/ROperator_Conv.hxx"
#include "SOFIE/ROperator_ConvTranspose.hxx"
#include "SOFIE/ROperator_Gemm.hxx"
#include "SOFIE/ROperator_Pool.hxx"
#include "SOFIE/ROperator_Quantized.hxx"
#include "SOFIE/ROperator_Relu.hxx"
#include "SOFIE/ROperator_Reshape.hxx"
