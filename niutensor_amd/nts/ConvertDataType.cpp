/*
 * Data type conversion of tensors on a gfx950 GPU.
 * Host logic of source/tensor/core/getandset/ConvertDataType.cpp:31-163: equal types return
 * at once, a GPU tensor goes to the GPU kernels (float <-> half, float <-> int; everything else
 * is "Unsupported data types for conversion!"), the allocating forms shape the result like
 * the input and record a GETANDSET_CONVERTDATATYPE edge when the input takes part in autograd.
 * Host tensors are refused: the reference's host code for half casts the value to an integer
 * (:95-106), and the CPU path is not part of this library anyway.
 */
#include "ConvertDataType.h"
#include "../../include/ntsamd_gemm.h"

namespace nts {

void _AmdConvertDataType(int devID, void * s, TENSOR_DATA_TYPE typeS, void * t, TENSOR_DATA_TYPE typeT, int size)
{
    CheckNTErrors((devID >= 0), "This code must be run on GPUs!");
    if (typeS == typeT)
        return;
    int rc = ntsamd_convert_data_type(devID, NULL, s, typeS, t, typeT, size);
    if (rc == NTSAMD_ERR_DATATYPE) {
        ShowNTErrors("Unsupported data types for conversion!");
    }
    else if (rc != NTSAMD_OK) {
        ShowNTErrors(ntsamd_last_error());
    }
}

void _ConvertDataType(const XTensor * input, XTensor * output)
{
    CheckNTErrors((input && output), "Empty input or output tensors!");
    if (input->dataType == output->dataType)
        return;
    CheckNTErrors((input->unitNum == output->unitNum), "Unmatched tensors!");
    if (input->devID >= 0) {
        CheckNTErrors((input->devID == output->devID), "The tensors must be on the same GPU!");
        _AmdConvertDataType(input->devID, input->data, input->dataType, output->data, output->dataType, input->unitNum);
        return;
    }
    ShowNTErrors("Host tensors are converted by NiuTensor's own CPU path, which this library does not replace!");
}

XTensor ConvertDataType(const XTensor & input, TENSOR_DATA_TYPE dataType)
{
    if (input.dataType == dataType) {
        /* the reference returns CopyValues(input) (:124-129) */
        XTensor output(input.order, input.dimSize, dataType, 1.0F, input.devID, input.mem);
        output.SetTMPFlag();
        XMemCopy(output.data, output.devID, input.data, input.devID, (size_t)input.unitNum * input.unitSize);
        return output;
    }

    XTensor output(input.order, input.dimSize, dataType, 1.0F, input.devID, input.mem);
    output.SetTMPFlag();

    _ConvertDataType(&input, &output);

    if (input.enableGrad)
        XLink::MakeLink(&input, NULL, &output, GETANDSET_CONVERTDATATYPE);

    return output;
}

void ConvertDataType(const XTensor & input, XTensor & output, TENSOR_DATA_TYPE dataType)
{
    if (!output.isInit || input.dataType != output.dataType)
        InitTensorV2(&output, input.order, input.dimSize, dataType, 1.0F, input.devID, input.mem);

    _ConvertDataType(&input, &output);

    if (input.enableGrad)
        XLink::MakeLink(&input, NULL, &output, GETANDSET_CONVERTDATATYPE);
}

}  // namespace nts
