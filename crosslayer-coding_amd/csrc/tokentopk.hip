// placeholder so the library links; replaced below
#include "clt_common.h"
extern "C" size_t clt_tokentopk_workspace_bytes(int64_t T, int64_t F, int64_t L, int64_t kk, int mode, int dtype) { return 256; }
extern "C" int clt_tokentopk_select(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride, int64_t kk, int mode, const float *mean, const float *denom, int dtype, int32_t *row_ptr, int32_t *col, void *val, void *workspace, size_t workspace_bytes, void *stream) { return CLT_ERR_ARG; }
