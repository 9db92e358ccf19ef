/*
 * Data-type and transpose enums with the reference's values
 * (source/tensor/XDataType.h:33,36). X_TRANS is 0 and X_NOTRANS is 1: the flag
 * is never a boolean "is transposed".
 */
#ifndef NTSAMD_XDATATYPE_H
#define NTSAMD_XDATATYPE_H

namespace nts {

enum TENSOR_DATA_TYPE { X_INT, X_INT8, X_FLOAT, X_FLOAT16, X_DOUBLE };
enum MATRIX_TRANS_TYPE { X_TRANS, X_NOTRANS };

#define DEFAULT_DTYPE X_FLOAT

inline int GetUnitSize(TENSOR_DATA_TYPE t)
{
    switch (t) {
    case X_INT: return 4;
    case X_INT8: return 1;
    case X_FLOAT: return 4;
    case X_FLOAT16: return 2;
    case X_DOUBLE: return 8;
    }
    return 0;
}

inline const char * GetDataTypeName(TENSOR_DATA_TYPE t)
{
    switch (t) {
    case X_INT: return "X_INT";
    case X_INT8: return "X_INT8";
    case X_FLOAT: return "X_FLOAT";
    case X_FLOAT16: return "X_FLOAT16";
    case X_DOUBLE: return "X_DOUBLE";
    }
    return "NULL";
}

}  // namespace nts
#endif
