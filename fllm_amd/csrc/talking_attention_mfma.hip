// Matrix-core forms of the attention whose heads talk to each other (talking_attention.hip says what is computed).
#include "api.h"
#include "common.h"

// 1: the shape is not taken, the caller runs the plain kernel
int fllm_talking_attention_bf16_fast(const void *q, const void *gate, int gate_stride, const void *k_pages, const void *v_pages,
                                     const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                                     const int32_t *seg_start, int num_segs, const float *talk, const float *temp, void *out,
                                     int rows, int heads, int kv_heads, int k_dim, int v_dim, int page_size, float scale, int chunk,
                                     int key_chunk, int max_context, hipStream_t stream) {
    return 1;
}
