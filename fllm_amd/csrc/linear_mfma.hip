#include "api.h"
#include "common.h"
int fllm_linear_bf16_fast(const void *, int, const void *, const float *, void *, int, int, int, int, int, hipStream_t) {
    return 1;
}
