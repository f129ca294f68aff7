/* Minimal declarations of the MATLAB MEX C API used by nnv_amd/matlab/nnvhip_mex.cpp, for a
 * syntax/type check of the gateway with g++ -fsyntax-only on machines without MATLAB.  It is not a
 * MATLAB replacement: nothing here is implemented or linked. */
#ifndef NNVHIP_TEST_MEX_STUB_H
#define NNVHIP_TEST_MEX_STUB_H
#include <cstddef>
#include <cstdint>
typedef struct mxArray_tag mxArray;
typedef size_t mwSize;
typedef enum { mxUINT64_CLASS = 13 } mxClassID;
typedef enum { mxREAL = 0 } mxComplexity;
extern "C" {
void mexErrMsgIdAndTxt(const char* id, const char* fmt, ...);
int mexAtExit(void (*fn)(void));
bool mxIsChar(const mxArray*);
bool mxIsDouble(const mxArray*);
bool mxIsComplex(const mxArray*);
bool mxIsEmpty(const mxArray*);
bool mxIsUint64(const mxArray*);
int mxGetString(const mxArray*, char*, mwSize);
double* mxGetDoubles(const mxArray*);
void* mxGetData(const mxArray*);
double mxGetScalar(const mxArray*);
size_t mxGetM(const mxArray*);
size_t mxGetN(const mxArray*);
size_t mxGetNumberOfElements(const mxArray*);
mwSize mxGetNumberOfDimensions(const mxArray*);
const mwSize* mxGetDimensions(const mxArray*);
mxArray* mxCreateDoubleMatrix(mwSize, mwSize, mxComplexity);
mxArray* mxCreateDoubleScalar(double);
mxArray* mxCreateNumericMatrix(mwSize, mwSize, mxClassID, mxComplexity);
void mxDestroyArray(mxArray*);
}
#endif
