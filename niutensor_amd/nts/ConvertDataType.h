/*
 * Data type conversion of tensors on a gfx950 GPU, with the reference's names
 * (source/tensor/core/getandset/ConvertDataType.h:31-45).
 */
#ifndef NTSAMD_CONVERTDATATYPE_H
#define NTSAMD_CONVERTDATATYPE_H

#include "XTensor.h"

namespace nts {

/* operation id of the autograd edge, value as in source/tensor/XName.h:88-93 */
#define DATA_BASE (MATH_BASE * 2)
#define GETANDSET (DATA_BASE + 1)
#define GETANDSET_CONVERTDATATYPE (GETANDSET + 1)

/* raw form: size elements of s (typeS) into t (typeT) on device devID */
void _AmdConvertDataType(int devID, void * s, TENSOR_DATA_TYPE typeS, void * t, TENSOR_DATA_TYPE typeT, int size);

/* output = (type of output) input, element by element; equal types do nothing */
void _ConvertDataType(const XTensor * input, XTensor * output);

/* a new tensor of type dataType (equal types: a copy of the values) */
XTensor ConvertDataType(const XTensor & input, TENSOR_DATA_TYPE dataType);

/* into `output`, which is formed on input's device when it is not yet or has a different type than input */
void ConvertDataType(const XTensor & input, XTensor & output, TENSOR_DATA_TYPE dataType);

}  // namespace nts
#endif
