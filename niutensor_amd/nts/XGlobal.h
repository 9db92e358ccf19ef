/*
 * Globals of the nts:: host layer: the element type and the fatal-error macros.
 * Same message format and same ending as the reference (source/tensor/XGlobal.h:78-102):
 * the message goes to stderr and a bare `throw;` follows, which ends the process
 * through std::terminate when no exception is in flight.
 */
#ifndef NTSAMD_XGLOBAL_H
#define NTSAMD_XGLOBAL_H

#include <stdio.h>
#include <string.h>

namespace nts {

/* source/tensor/XGlobal.h:48-56: DOUBELPRICSION is not defined, so DTYPE is float */
#define DTYPE float

#define NTS_FILENAME (strrchr(__FILE__, '/') ? strrchr(__FILE__, '/') + 1 : __FILE__)

#define CheckNTErrors(x, msg) \
{ \
    if (!(x)) \
    { \
        fprintf(stderr, "[ERROR] calling '%s' (%s line %d): %s\n", #x, NTS_FILENAME, __LINE__, msg); \
        fflush(stderr); \
        throw; \
    } \
}

#define ShowNTErrors(msg) \
{ \
    { \
        fprintf(stderr, "[ERROR] (%s line %d): %s\n", NTS_FILENAME, __LINE__, msg); \
        fflush(stderr); \
        throw; \
    } \
}

#ifndef MAX
#define MAX(a, b) ((a) > (b) ? (a) : (b))
#endif

/* the thread-pool handle of the CPU path; the GPU path never looks at it */
struct XPRunner;

}  // namespace nts
#endif
