/*
 * C ABI of the MI355X convolution / pooling / normalisation backend
 * (libcudamat_conv.so).  Names, argument order and argument meaning are those of
 * the 13 exports of the reference's cudamat/cudamat_conv.cu:1402-1456, which
 * cudamat/cudamat_conv.py binds through ctypes.  These 13, the two fused pooling +
 * normalisation calls at the end and conv_last_error are the library's whole dynamic symbol table.  It links against libcudamat.so (found next to it),
 * whose stream, workspaces and block cache it shares: calls of both libraries run in call
 * order on one stream and are recorded into the same HIP graphs.
 *
 * Layout (cudamat/cudamat_conv.cu:9-13): every operand is a column-major cudamat
 * whose size[0] is the number of images, so the flat index of pixel (c, y, x) of
 * image n is  n + numImages * ((c * imgSize + y) * imgSize + x)  - cuda-convnet's
 * (channels, rows, cols, batch) with the batch fastest.  Filters are
 * (numFilters, filterColors * filterSize^2) matrices: f + numFilters * ((c * k + ky) * k + kx).
 *
 * All entry points return void like the reference's.  Where the reference
 * aborts the process on a bad shape (C assert), these record a message instead:
 * conv_last_error() returns it (NULL when the last call succeeded) and the
 * Python wrapper raises.
 */
#ifndef CUDAMAT_CONV_AMD_H_
#define CUDAMAT_CONV_AMD_H_

#include "cudamat_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference (it asserts): message of the last failed call, or NULL. */
const char* conv_last_error(void);

/* ---- shared-filter convolution: cudamat_conv.cu:1404-1412 (filterActs :15-257, imgActs :265-640,
 * weightActs :642-1015).  paddingStart is <= 0 (the Python wrapper negates it). ---- */
void convUp(cudamat* images, cudamat* filters, cudamat* targets, int numModulesX, int paddingStart, int moduleStride,
            int numImgColors, int numGroups);
void convDown(cudamat* hidActs, cudamat* filters, cudamat* targets, int imgSize, int paddingStart, int moduleStride,
              int numImgColors, int numGroups);
void convOutp(cudamat* images, cudamat* hidActs, cudamat* targets, int numModulesX, int filterSize, int paddingStart,
              int moduleStride, int numImgColors, int numGroups, int partialSum);

/* ---- locally connected (unshared filters): cudamat_conv.cu:1415-1423 ---- */
void localUp(cudamat* images, cudamat* filters, cudamat* targets, int numModulesX, int paddingStart, int moduleStride,
             int numImgColors, int numGroups);
void localDown(cudamat* hidActs, cudamat* filters, cudamat* targets, int imgSize, int paddingStart, int moduleStride,
               int numImgColors, int numGroups);
void localOutp(cudamat* images, cudamat* hidActs, cudamat* targets, int numModulesX, int filterSize, int paddingStart,
               int moduleStride, int numImgColors, int numGroups, int partialSum);

/* ---- response / contrast normalisation: cudamat_conv.cu:1426-1439 (convContrastNorm
 * cudamat_conv_kernels.cu:303-441, convResponseNormUndo cudamat_conv.cu:1291-1387).
 * ResponseNormUndo overwrites `acts` with -2*addScale*powScale*outGrads*acts/denoms. ---- */
void ResponseNorm(cudamat* images, cudamat* denoms, cudamat* targets, int numFilters, int sizeX, float addScale,
                  float powScale);
void ResponseNormUndo(cudamat* outGrads, cudamat* denoms, cudamat* inputs, cudamat* acts, cudamat* targets,
                      int numFilters, int sizeX, float addScale, float powScale);
void ContrastNorm(cudamat* images, cudamat* meanDiffs, cudamat* denoms, cudamat* targets, int numFilters, int sizeX,
                  float addScale, float powScale);
void ContrastNormUndo(cudamat* outGrads, cudamat* denoms, cudamat* meanDiffs, cudamat* acts, cudamat* targets,
                      int numFilters, int sizeX, float addScale, float powScale);

/* ---- local pooling: cudamat_conv.cu:1442-1454 (convLocalPool :1021-1120, convLocalProbPool
 * :1189-1289, convLocalMaxUndo :1128-1182).  MaxPool may be held back (unless
 * set_deferred_epilogues(0) of libcudamat.so is in force): a ResponseNorm of its target that follows
 * directly runs with it as one launch, any other call of either library launches it first; same
 * results in every array. ---- */
void MaxPool(cudamat* images, cudamat* targets, int numFilters, int subsX, int startX, int strideX, int outputsX);
void ProbMaxPool(cudamat* images, cudamat* rnd, cudamat* targets, int numFilters, int subsX, int startX, int strideX,
                 int outputsX);
void MaxPoolUndo(cudamat* images, cudamat* maxGrads, cudamat* maxActs, cudamat* targets, int subsX, int startX,
                 int strideX, int outputsX);

/* ---- Extensions (no counterpart in the reference): the two pairs of calls that deepnet/convolutions.py:58-66
 * and :120-134 always issue back to back, each in one launch (the pooled map of a block of images stays in LDS
 * between the two stages); results are those of the separate calls.
 * MaxPoolResponseNorm: pooled = MaxPool(images); (denoms, targets) = ResponseNorm(pooled).
 * ResponseNormUndoMaxPoolUndo: targets = MaxPoolUndo(images, maxGrads = ResponseNormUndo(outGrads, denoms, inputs,
 * acts), maxActs = acts); `acts` (the pooled activations) is left unchanged; targets may be images. ---- */
void MaxPoolResponseNorm(cudamat* images, cudamat* pooled, cudamat* denoms, cudamat* targets, int numFilters, int subsX,
                         int startX, int strideX, int outputsX, int sizeX, float addScale, float powScale);
void ResponseNormUndoMaxPoolUndo(cudamat* outGrads, cudamat* denoms, cudamat* inputs, cudamat* acts, cudamat* images,
                                 cudamat* targets, int numFilters, int subsX, int startX, int strideX, int outputsX, int sizeX,
                                 float addScale, float powScale);

#ifdef __cplusplus
}
#endif
#endif /* CUDAMAT_CONV_AMD_H_ */
