// temporary: entry points not written yet
#include "common.h"
#define STUB(name, ...) extern "C" int name(__VA_ARGS__) { ::dh::set_error(__FILE__, __LINE__, __func__, "not implemented yet"); return DH_ERR_UNSUPPORTED; }
STUB(dh_moe_route_topk, const float *logits, int32_t *topk_idx, float *gates, int64_t tokens, int experts, int k, void *stream)
extern "C" size_t dh_moe_sort_workspace_bytes(int64_t n_assign, int experts) { return 16; }
STUB(dh_moe_sort, const int32_t *topk_idx, int32_t *tokens_per_expert, int32_t *sorted_idx, int32_t *dest_row, void *workspace, int64_t n_assign, int experts, void *stream)
STUB(dh_moe_gather_rows, const void *x, const int32_t *src_assign, const float *row_scale, void *permuted, const int32_t *n_rows_dev, int64_t max_rows, int k, int64_t hidden, int dtype, void *stream)
STUB(dh_moe_scatter_rows, const void *y, const int32_t *dest_row, const float *gates, void *out, const int32_t *range_dev, int64_t tokens, int k, int64_t hidden, int dtype, void *stream)
STUB(dh_moe_gate_grad, const void *dout, const void *y, const int32_t *dest_row, float *dgates, const int32_t *range_dev, int64_t tokens, int k, int64_t hidden, int dtype, void *stream)
STUB(dh_grouped_gemm_nt, const void *a, const void *b, void *c, const int32_t *offs, int groups, int64_t max_rows, int64_t n, int64_t k, int dtype, void *stream)
STUB(dh_grouped_gemm_nn, const void *a, const void *b, void *c, const int32_t *offs, int groups, int64_t max_rows, int64_t n, int64_t k, int dtype, void *stream)
STUB(dh_grouped_gemm_tn, const void *a, const void *b, void *c, const int32_t *offs, int groups, int64_t max_rows, int64_t m, int64_t n, int accumulate, int dtype, void *stream)
