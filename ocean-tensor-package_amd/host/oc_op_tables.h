/* Entries of the core-module function table that are generated from lists in the reference
 * (include/ocean/core/generic/generate_tensor_unary.h:19-62, generate_tensor_binary.h:19-47, the axis
 * reductions of include/ocean/core/interface/module_core.h:126-152), each with the operation index that the
 * device library (include/ocean_hip.h) uses for it. X(table entry name, och operation index). */
#ifndef OC_OP_TABLES_H
#define OC_OP_TABLES_H
#define OC_UNARY_TABLE(X) \
   X(negative, 0) X(bitwiseNot, 1) X(logicalNot, 2) X(conj, 3) X(reciprocal, 4) X(sin, 5) X(cos, 6) X(tan, 7) \
   X(sinh, 8) X(cosh, 9) X(tanh, 10) X(arcsin, 11) X(arccos, 12) X(arctan, 13) X(arcsinh, 14) X(arccosh, 15) \
   X(arctanh, 16) X(sqrt, 17) X(cbrt, 18) X(square, 19) X(exp, 20) X(exp2, 21) X(exp10, 22) X(expm1, 23) \
   X(log, 24) X(log2, 25) X(log10, 26) X(log1p, 27) X(absolute, 28) X(fabs, 29) X(sign, 30) X(ceil, 31) \
   X(floor, 32) X(trunc, 33) X(round, 34) X(isinf, 35) X(isnan, 36) X(isfinite, 37) X(isposinf, 38) X(isneginf, 39)
#define OC_BINARY_TABLE(X) \
   X(add, 0) X(subtract, 1) X(scale, 2) X(divide, 3) X(trueDivide, 4) X(floorDivide, 5) X(power, 6) X(mod, 7) X(fmod, 8) \
   X(elemwiseMin, 9) X(elemwiseMax, 10) X(elemwiseFMin, 11) X(elemwiseFMax, 12) X(elemwiseLT, 13) X(elemwiseLE, 14) \
   X(elemwiseEQ, 15) X(elemwiseNE, 16) X(elemwiseGE, 17) X(elemwiseGT, 18) X(bitwiseAnd, 19) X(bitwiseOr, 20) \
   X(bitwiseXor, 21) X(logicalAnd, 22) X(logicalOr, 23) X(logicalXor, 24) X(bitshiftLeft, 25) X(bitshiftRight, 26)
/* axis reductions in table order; X(table name, och reduction index) */
#define OC_AXIS_TABLE(X) \
   X(axisAny, 0) X(axisAll, 1) X(axisAllFinite, 2) X(axisAnyInf, 3) X(axisAnyNaN, 4) X(axisNnz, 5) X(axisNnzNaN, 6) \
   X(axisSum, 15) X(axisProd, 17) X(axisSumNaN, 16) X(axisProdNaN, 18) X(axisSumAbs, 19) X(axisSumAbsNaN, 20) \
   X(axisMinimum, 22) X(axisMaximum, 21) X(axisMinimumAbs, 24) X(axisMaximumAbs, 23) X(axisNorm2, 27) X(axisNorm2NaN, 28)

#endif
