// Attention whose heads talk to each other before the softmax, over the paged cache, plain form.
//
//   raw[g](row, key)  = q_g(row) . k_{g / group}(key) * scale * temp[g]
//   s[h](row, key)    = sum_g talk[h, g] * raw[g](row, key)              (every head's score is a mix of all heads' scores)
//   p[h]              = softmax of s[h] over the keys the row sees
//   out[h](row)       = gate[h](row) * sum_key p[h](row, key) * v_{h / group}(key)
//
// A row at position pos sees the keys lo .. pos of its request, lo = pos - pos % chunk (chunk 0: lo = 0): chunks are
// counted from the request's first position.  Keys and values may have different widths.  One workgroup a row holds all
// heads of that row, because the mix needs every head's score of a key at once.  float32 arithmetic; a row's result
// depends on its own position and pages alone, never on the rest of the batch.
//
// The kernel before it (qk_norm_rope_store) takes the rows of the joint q/k/v product: an RMSNorm over the whole query
// projection and one over the whole key projection (all heads at once, a weight a lane), rotary on the first
// rope_dims lanes of every head (lane i paired with lane i + rope_dims / 2), queries out, keys and values into pages.
#include "api.h"
#include "common.h"

int fllm_talking_attention_bf16_fast(const void *q, const void *gate, int gate_stride, const void *k_pages, const void *v_pages,
                                     const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                                     const int32_t *seg_start, int num_segs, const float *talk, const float *temp, void *out,
                                     int rows, int heads, int kv_heads, int k_dim, int v_dim, int page_size, float scale, int chunk,
                                     int key_chunk, int max_context, int splits, float *ws, size_t ws_floats, int single_rows,
                                     hipStream_t stream);   // talking_attention_mfma.hip; 1: declined

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
constexpr int kMaxOut = 16;   // heads * v_dim <= kBlock * kMaxOut

// [page][kv_head][k_dim / c][token][c]: c = 8 is key_offset() of common.h, c = 1 keys transposed like the values
__device__ __forceinline__ size_t key_at(size_t page, int kv_heads, int kvh, int page_size, int k_dim, int token, int d, int c) {
    return ((((size_t)page * kv_heads + kvh) * (k_dim / c) + d / c) * page_size + token) * c + d % c;
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
qk_norm_rope_store_kernel(const T *__restrict__ qkv, int ld, const float *__restrict__ q_weight, const float *__restrict__ k_weight,
                          float eps, T *__restrict__ q_out, const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg,
                          const int32_t *__restrict__ tables, int table_stride, const float *__restrict__ cos_table,
                          const float *__restrict__ sin_table, T *__restrict__ k_pages, T *__restrict__ v_pages, int heads,
                          int kv_heads, int k_dim, int v_dim, int rope_dims, int page_size, int key_chunk, int store_kv) {
    __shared__ float scratch[kWaves];
    const size_t r = blockIdx.x;
    const int seg = row_seg[r];
    if (seg < 0) return;   // padding row: its queries are never read
    const int pos = row_pos[r];
    const int nq = heads * k_dim, nk = kv_heads * k_dim, nv = kv_heads * v_dim;
    const T *q = qkv + r * ld, *k = q + nq, *v = k + nk;
    // asked for before the sums, so that the lookup waits beside them and not behind them
    const int page = store_kv ? tables[(size_t)seg * table_stride + pos / page_size] : 0, off = pos % page_size;
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < nq; c += kBlock) { const float a = to_f32<T>(q[c]); sq += a * a; }
    for (int c = threadIdx.x; c < nk; c += kBlock) { const float a = to_f32<T>(k[c]); sk += a * a; }
    sq = block_sum<kWaves>(sq, scratch);
    sk = block_sum<kWaves>(sk, scratch);
    const float inv_q = 1.0f / sqrtf(sq / (float)nq + eps), inv_k = 1.0f / sqrtf(sk / (float)nk + eps);
    const int half = rope_dims / 2;
    const float *cs = cos_table + (size_t)pos * half, *sn = sin_table + (size_t)pos * half;
    for (int idx = threadIdx.x; idx < nq + (store_kv ? nk : 0); idx += kBlock) {
        const bool is_q = idx < nq;
        const int e = is_q ? idx : idx - nq;
        const T *src = is_q ? q : k;
        const float *w = is_q ? q_weight : k_weight;
        const float inv = is_q ? inv_q : inv_k;
        const int h = e / k_dim, c = e - h * k_dim;
        float val = to_f32<T>(src[e]) * inv * w[e];
        if (c < rope_dims) {
            const int i = c < half ? c : c - half;
            const int pe = c < half ? e + half : e - half;
            const float other = to_f32<T>(src[pe]) * inv * w[pe];
            val = c < half ? val * cs[i] - other * sn[i] : val * cs[i] + other * sn[i];
        }
        if (is_q) q_out[r * nq + e] = from_f32<T>(val);
        else k_pages[key_at(page, kv_heads, h, page_size, k_dim, off, c, key_chunk)] = from_f32<T>(val);
    }
    if (!store_kv) return;
    for (int e = threadIdx.x; e < nv; e += kBlock) {
        const int h = e / v_dim, c = e - h * v_dim;
        v_pages[(((size_t)page * kv_heads + h) * v_dim + c) * page_size + off] = v[e];
    }
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
talking_attention_kernel(const T *__restrict__ q, const T *__restrict__ gate, int gate_stride, const T *__restrict__ k_pages,
                         const T *__restrict__ v_pages, const int32_t *__restrict__ tables, int table_stride,
                         const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg, const float *__restrict__ talk,
                         const float *__restrict__ temp, T *__restrict__ out, int heads, int kv_heads, int k_dim, int v_dim,
                         int page_size, float scale, int chunk, int key_chunk) {
    extern __shared__ float smem[];
    float *qs = smem;                         // heads * k_dim, already times scale * temp[head]
    float *raw = qs + heads * k_dim;          // heads * kBlock
    float *sc = raw + heads * kBlock;         // heads * kBlock: mixed scores, then weights
    float *tk = sc + heads * kBlock;          // heads * heads
    float *run_m = tk + heads * heads;        // heads
    float *run_l = run_m + heads;             // heads
    float *alpha = run_l + heads;             // heads
    const size_t r = blockIdx.x;
    const int seg = row_seg[r];
    const int total = heads * v_dim;
    T *dst = out + r * total;
    if (seg < 0) {   // padding row
        for (int c = threadIdx.x; c < total; c += kBlock) dst[c] = from_f32<T>(0.f);
        return;
    }
    const int pos = row_pos[r];
    const int n = pos + 1;
    const int lo = chunk > 0 ? pos - pos % chunk : 0;
    const int group = heads / kv_heads;
    const int32_t *tbl = tables + (size_t)seg * table_stride;
    for (int c = threadIdx.x; c < heads * k_dim; c += kBlock) qs[c] = to_f32<T>(q[r * heads * k_dim + c]) * (scale * temp[c / k_dim]);
    for (int c = threadIdx.x; c < heads * heads; c += kBlock) tk[c] = talk[c];
    for (int c = threadIdx.x; c < heads; c += kBlock) { run_m[c] = -INFINITY; run_l[c] = 0.f; }
    __syncthreads();

    float acc[kMaxOut];
#pragma unroll
    for (int t = 0; t < kMaxOut; t++) acc[t] = 0.f;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    for (int c0 = lo; c0 < n; c0 += kBlock) {
        const int key = c0 + threadIdx.x;
        if (key < n) {
            const int page = tbl[key / page_size], off = key % page_size;
            for (int kvh = 0; kvh < kv_heads; kvh++) {
                for (int g = kvh * group; g < (kvh + 1) * group; g++) {
                    const float *qg = qs + g * k_dim;
                    float dot = 0.f;
                    for (int c = 0; c < k_dim; c++)
                        dot = fmaf(qg[c], to_f32<T>(k_pages[key_at(page, kv_heads, kvh, page_size, k_dim, off, c, key_chunk)]), dot);
                    raw[g * kBlock + threadIdx.x] = dot;
                }
            }
            for (int h = 0; h < heads; h++) {   // the thread reads back what it wrote itself
                float s = 0.f;
                for (int g = 0; g < heads; g++) s = fmaf(tk[h * heads + g], raw[g * kBlock + threadIdx.x], s);
                sc[h * kBlock + threadIdx.x] = s;
            }
        } else {
            for (int h = 0; h < heads; h++) sc[h * kBlock + threadIdx.x] = -INFINITY;
        }
        __syncthreads();
        // a wave a head: largest score of the chunk, weights, their sum
        for (int h = wave; h < heads; h += kWaves) {
            float *row = sc + h * kBlock;
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < kBlock / kWave; j++) mx = fmaxf(mx, row[lane + j * kWave]);
            const float m_old = run_m[h];
            const float m_new = fmaxf(m_old, wave_max(mx));
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < kBlock / kWave; j++) {
                const float p = expf(row[lane + j * kWave] - m_new);   // exp(-inf) = 0 for keys beyond the row's last
                row[lane + j * kWave] = p;
                sum += p;
            }
            sum = wave_sum(sum);
            if (lane == 0) {
                const float a = expf(m_old - m_new);   // first chunk: exp(-inf) = 0
                alpha[h] = a;
                run_l[h] = run_l[h] * a + sum;
                run_m[h] = m_new;
            }
        }
        __syncthreads();
        const int count = n - c0 < kBlock ? n - c0 : kBlock;
#pragma unroll
        for (int t = 0; t < kMaxOut; t++) {
            const int o = threadIdx.x + t * kBlock;
            if (o >= total) break;
            const int h = o / v_dim, c = o - h * v_dim, kvh = h / group;
            const float *p = sc + h * kBlock;
            float a = acc[t] * alpha[h];
            for (int j = 0; j < count; j++) {
                const int kj = c0 + j;
                const int page = tbl[kj / page_size], off = kj % page_size;
                a = fmaf(p[j], to_f32<T>(v_pages[(((size_t)page * kv_heads + kvh) * v_dim + c) * page_size + off]), a);
            }
            acc[t] = a;
        }
        __syncthreads();   // sc[] and alpha[] are rewritten by the next chunk
    }
#pragma unroll
    for (int t = 0; t < kMaxOut; t++) {
        const int o = threadIdx.x + t * kBlock;
        if (o >= total) break;
        const int h = o / v_dim;
        float val = acc[t] / run_l[h];
        if (gate != nullptr) val *= 1.0f / (1.0f + expf(-to_f32<T>(gate[r * gate_stride + h])));
        dst[o] = from_f32<T>(val);
    }
}

size_t plain_lds_bytes(int heads, int k_dim) {
    return (size_t)(heads * k_dim + 2 * heads * kBlock + heads * heads + 3 * heads) * sizeof(float);
}

}  // namespace

extern "C" int fllm_qk_norm_rope_store(const void *qkv, int ld, const float *q_weight, const float *k_weight, float eps, void *q_out,
                                       const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables, int table_stride,
                                       const float *cos_table, const float *sin_table, int table_positions, void *k_pages,
                                       void *v_pages, int rows, int heads, int kv_heads, int k_dim, int v_dim, int rope_dims,
                                       int page_size, int key_chunk, int dtype, int store_kv, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && kv_heads > 0 && k_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0,
                 "qk_norm_rope_store: bad sizes");
    FLLM_REQUIRE(ld >= heads * k_dim + kv_heads * (k_dim + v_dim), "qk_norm_rope_store: rows of %d values cannot hold q, k and v", ld);
    FLLM_REQUIRE(rope_dims >= 0 && rope_dims <= k_dim && rope_dims % 2 == 0,
                 "qk_norm_rope_store: rope_dims %d must be even and at most the head size %d", rope_dims, k_dim);
    FLLM_REQUIRE(rope_dims == 0 || (cos_table && sin_table && table_positions > 0), "qk_norm_rope_store: rotary tables missing");
    FLLM_REQUIRE(key_chunk > 0 && k_dim % key_chunk == 0, "qk_norm_rope_store: keys of %d values in chunks of %d", k_dim, key_chunk);
    FLLM_REQUIRE(!store_kv || (k_pages && v_pages), "qk_norm_rope_store: pages missing");
    FLLM_REQUIRE(q_weight && k_weight && q_out, "qk_norm_rope_store: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(qk_norm_rope_store_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, (const float *)qkv, ld, q_weight,
                           k_weight, eps, (float *)q_out, row_pos, row_seg, tables, table_stride, cos_table, sin_table,
                           (float *)k_pages, (float *)v_pages, heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk, store_kv);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(qk_norm_rope_store_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, (const bf16_t *)qkv, ld, q_weight,
                           k_weight, eps, (bf16_t *)q_out, row_pos, row_seg, tables, table_stride, cos_table, sin_table,
                           (bf16_t *)k_pages, (bf16_t *)v_pages, heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk,
                           store_kv);
    else
        FLLM_REQUIRE(false, "qk_norm_rope_store: unknown dtype %d", dtype);
    return fllm_check_launch("qk_norm_rope_store");
}

extern "C" int fllm_talking_attention(const void *q, const void *gate, int gate_stride, const void *k_pages, const void *v_pages,
                                      const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                                      const int32_t *seg_start, int num_segs, const float *talk, const float *temp, void *out,
                                      int rows, int heads, int kv_heads, int k_dim, int v_dim, int page_size, float scale,
                                      int chunk, int key_chunk, int dtype, int max_context, int splits, float *ws, size_t ws_floats,
                                      int single_rows, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && kv_heads > 0 && k_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0,
                 "talking_attention: bad sizes");
    FLLM_REQUIRE(heads % kv_heads == 0, "talking_attention: %d heads are not a multiple of %d key/value heads", heads, kv_heads);
    FLLM_REQUIRE(chunk >= 0, "talking_attention: chunk %d", chunk);
    FLLM_REQUIRE(key_chunk > 0 && k_dim % key_chunk == 0, "talking_attention: keys of %d values in chunks of %d", k_dim, key_chunk);
    FLLM_REQUIRE(talk && temp && q && out && k_pages && v_pages, "talking_attention: operands missing");
    FLLM_REQUIRE(gate == nullptr || gate_stride >= heads, "talking_attention: gate rows of %d values for %d heads", gate_stride, heads);
    if (rows == 0) return 0;
    if (dtype == FLLM_BF16 && fllm_fast_kernels_enabled()) {
        const int fast = fllm_talking_attention_bf16_fast(q, gate, gate_stride, k_pages, v_pages, tables, table_stride, row_pos, row_seg,
                                                          seg_start, num_segs, talk, temp, out, rows, heads, kv_heads, k_dim, v_dim,
                                                          page_size, scale, chunk, key_chunk, max_context, splits, ws, ws_floats, single_rows, stream);
        if (fast <= 0) return fast;
    }
    FLLM_REQUIRE(heads * v_dim <= kBlock * kMaxOut, "talking_attention: %d heads of %d values are more than %d outputs a row", heads,
                 v_dim, kBlock * kMaxOut);
    const size_t lds = plain_lds_bytes(heads, k_dim);
    FLLM_REQUIRE(lds <= 160 * 1024, "talking_attention: %d heads of %d values need %zu bytes of LDS", heads, k_dim, lds);
    if (dtype == FLLM_F32) {
        if (lds > 48 * 1024)
            FLLM_REQUIRE(hipFuncSetAttribute((const void *)talking_attention_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)lds) == hipSuccess, "talking_attention: cannot have %zu bytes of LDS", lds);
        hipLaunchKernelGGL(talking_attention_kernel<float>, dim3(rows), dim3(kBlock), lds, stream, (const float *)q, (const float *)gate,
                           gate_stride, (const float *)k_pages, (const float *)v_pages, tables, table_stride, row_pos, row_seg, talk,
                           temp, (float *)out, heads, kv_heads, k_dim, v_dim, page_size, scale, chunk, key_chunk);
    } else if (dtype == FLLM_BF16) {
        if (lds > 48 * 1024)
            FLLM_REQUIRE(hipFuncSetAttribute((const void *)talking_attention_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)lds) == hipSuccess, "talking_attention: cannot have %zu bytes of LDS", lds);
        hipLaunchKernelGGL(talking_attention_kernel<bf16_t>, dim3(rows), dim3(kBlock), lds, stream, (const bf16_t *)q,
                           (const bf16_t *)gate, gate_stride, (const bf16_t *)k_pages, (const bf16_t *)v_pages, tables, table_stride,
                           row_pos, row_seg, talk, temp, (bf16_t *)out, heads, kv_heads, k_dim, v_dim, page_size, scale, chunk,
                           key_chunk);
    } else {
        FLLM_REQUIRE(false, "talking_attention: unknown dtype %d", dtype);
    }
    return fllm_check_launch("talking_attention");
}
