/* Plain C client of the model_calcer C ABI (include/c_api.h), the way a program written against the
 * reference's libcatboostmodel calls it. Usage: c_abi_client model.cbm f0 f1 f2 ...  -> prints the prediction. */
#include "../include/c_api.h"

#include <stdio.h>
#include <stdlib.h>

int main(int argc, char** argv) {
    if (argc < 3) {
        fprintf(stderr, "usage: %s model.cbm feature...\n", argv[0]);
        return 2;
    }
    ModelCalcerHandle* h = ModelCalcerCreate();
    if (!h || !LoadFullModelFromFile(h, argv[1])) {
        fprintf(stderr, "load failed: %s\n", GetErrorString());
        return 1;
    }
    if (!EnableGPUEvaluation(h, 0)) {
        fprintf(stderr, "EnableGPUEvaluation failed: %s\n", GetErrorString());
        return 1;
    }
    size_t n = (size_t)(argc - 2);
    float* row = (float*)malloc(sizeof(float) * n);
    for (size_t i = 0; i < n; ++i) {
        row[i] = (float)atof(argv[2 + i]);
    }
    const float* rows[1] = {row};
    size_t dims = GetPredictionDimensionsCount(h);
    double* out = (double*)malloc(sizeof(double) * dims);
    if (!CalcModelPredictionFlat(h, 1, rows, n, out, dims)) {
        fprintf(stderr, "predict failed: %s\n", GetErrorString());
        return 1;
    }
    for (size_t k = 0; k < dims; ++k) {
        printf("%.17g\n", out[k]);
    }
    free(out);
    free(row);
    ModelCalcerDelete(h);
    return 0;
}
