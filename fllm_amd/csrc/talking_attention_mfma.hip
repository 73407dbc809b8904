// Matrix-core form of the attention whose heads talk to each other (talking_attention.hip says what is computed),
// bfloat16 operands, float32 scores, statistics and sums.
//
// A workgroup of four waves takes 16 consecutive rows of one request (a prompt portion's row tile, or a decode step's
// single row) with ALL heads, because a mixed score needs every head's raw score of the same (row, key).  It walks the
// keys the tile sees in blocks of 64.  The products are the transposed ones, v_mfma_f32_16x16x32_bf16 with
// D[m = 4 (l / 16) + i][n = l % 16], so that a lane keeps one row throughout:
//
//   1. wave w takes the block's keys 16 w .. 16 w + 15: for every head  raw_g^T[key][row] = K_{g / group} Q_g^T
//      (A = 16 keys x 32 lanes straight from the pages, B = the rows' queries from LDS).  A lane then holds, for its four
//      (key, row) pairs, the raw scores of all heads: the mix  s_h = sum_g talk'[h, g] raw_g  is lane-local
//      (talk'[h, g] = talk[h, g] * scale * temp[g], prepared in LDS once).
//   2. the block's largest score a (head, row) goes through LDS (four waves hold different keys); every wave computes
//      the same running maximum, weighs its scores, keeps its share of the running sum and leaves the weights in LDS
//      as bfloat16, [head][key group][row][16 keys].
//   3. the outputs  O_h^T[lane of v][row] += V_{h / group}^T P_h^T  are dealt out to the waves by (head, 16 value lanes):
//      B = weights from LDS, A = values from the pages, whose transposed order makes a lane's four keys 8 bytes in a row.
//      The k slots of this product hold the keys 4 g + i of two key groups, the order step 2 left them in.
//
// Rows of a tile see different key ranges when a chunk of positions ends inside the tile: the mask is per (row, key).
#include "api.h"
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kTileRows = 16;
constexpr int kKeyBlock = 64;

struct TalkArgs {
    const bf16_t *q, *gate;
    int gate_stride;
    const bf16_t *k_pages, *v_pages;
    const int32_t *tables;
    int table_stride;
    const int32_t *row_pos, *row_seg, *seg_start;
    int num_segs;
    const float *talk, *temp;
    bf16_t *out;
    int rows, heads, kv_heads, k_dim, v_dim, page_size;
    float scale;
    int chunk;
};

template <int HMAX, int KSMAX, int UMAX>
__global__ void __launch_bounds__(kThreads)
talking_tile_kernel(const TalkArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    __shared__ float tk[HMAX * HMAX];
    __shared__ float mx[4][HMAX][kTileRows];
    __shared__ float al[HMAX][kTileRows];
    __shared__ __attribute__((aligned(16))) bf16_t ps[HMAX][4][kTileRows][16];
    bf16_t *qs = (bf16_t *)lds_raw;

    const int H = p.heads, G = p.kv_heads, D = p.k_dim, DV = p.v_dim, PS = p.page_size;
    const int group = H / G, KS = D / 32, DVT = DV / 16;
    const int QP = H * D + 8;
    // which rows: the workgroup's tile among the tiles of all segments
    int seg = -1, first = 0, nrows = 0;
    {
        int before = 0;
        for (int s = 0; s < p.num_segs; s++) {
            const int r0 = p.seg_start[s], n = p.seg_start[s + 1] - r0;
            const int tiles = (n + kTileRows - 1) / kTileRows;
            if ((int)blockIdx.x < before + tiles) {
                const int t = blockIdx.x - before;
                seg = s;
                first = r0 + t * kTileRows;
                nrows = n - t * kTileRows < kTileRows ? n - t * kTileRows : kTileRows;
                break;
            }
            before += tiles;
        }
    }
    if (seg < 0) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const size_t out_row = (size_t)H * DV;
    if (p.row_seg[first] < 0) {   // padding rows of a captured step
        for (int i = threadIdx.x; i < nrows * H * DV; i += kThreads) p.out[(size_t)first * out_row + i] = (bf16_t)0.f;
        return;
    }
    const int pos0 = p.row_pos[first], plast = pos0 + nrows - 1;
    const int lo_tile = p.chunk > 0 ? pos0 - pos0 % p.chunk : 0;
    const int kb_start = lo_tile & ~15;
    const int32_t *tbl = p.tables + (size_t)seg * p.table_stride;
    const int pos_c = c < nrows ? pos0 + c : -1;
    const int lo_c = p.chunk > 0 && pos_c >= 0 ? pos_c - pos_c % p.chunk : 0;

    // queries of the tile and the mixing matrix into LDS
    {
        const int per_row = H * D / 8;
        for (int i = threadIdx.x; i < kTileRows * per_row; i += kThreads) {
            const int r = i / per_row, e = (i - r * per_row) * 8;
            bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (r < nrows) v = *(const bf16x8_t *)(p.q + (size_t)(first + r) * H * D + e);
            *(bf16x8_t *)(qs + r * QP + e) = v;
        }
        for (int i = threadIdx.x; i < HMAX * HMAX; i += kThreads) {
            const int h = i / HMAX, gg = i % HMAX;
            tk[i] = h < H && gg < H ? p.talk[h * H + gg] * (p.scale * p.temp[gg]) : 0.f;
        }
    }
    __syncthreads();

    float m_run[HMAX], l_part[HMAX];
    f32x4_t o[UMAX];
#pragma unroll
    for (int h = 0; h < HMAX; h++) { m_run[h] = -INFINITY; l_part[h] = 0.f; }
#pragma unroll
    for (int j = 0; j < UMAX; j++) o[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    const int units = H * DVT;

    for (int kb = kb_start; kb <= plast; kb += kKeyBlock) {
        // ---- 1. raw scores of this wave's 16 keys for every head, then the mix
        f32x4_t s[HMAX];
        const int key0 = kb + 16 * wave;
        const bool active = key0 <= plast;      // wave-uniform
        if (active) {
            f32x4_t raw[HMAX];
            const int key_a = key0 + c <= plast ? key0 + c : plast;      // the key of this lane's A row (clamped: masked later)
            const int page = tbl[key_a / PS], off = key_a % PS;
            bf16x8_t kf[KSMAX];
            int loaded = -1;
#pragma unroll
            for (int h = 0; h < HMAX; h++) {
                raw[h] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                if (h < H) {
                    const int kvh = h / group;
                    if (kvh != loaded) {
                        loaded = kvh;
#pragma unroll
                        for (int ks = 0; ks < KSMAX; ks++)
                            if (ks < KS) kf[ks] = *(const bf16x8_t *)(p.k_pages + key_offset(page, G, kvh, PS, D, off, 32 * ks + 8 * g));
                    }
#pragma unroll
                    for (int ks = 0; ks < KSMAX; ks++)
                        if (ks < KS) {
                            const bf16x8_t qf = *(const bf16x8_t *)(qs + c * QP + h * D + 32 * ks + 8 * g);
                            raw[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf, raw[h], 0, 0, 0);
                        }
                }
            }
            bool see[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = key0 + 4 * g + i;
                see[i] = key >= lo_c && key <= pos_c;
            }
#pragma unroll
            for (int h = 0; h < HMAX; h++) {
                f32x4_t v = {0.f, 0.f, 0.f, 0.f};
                if (h < H) {
#pragma unroll
                    for (int gg = 0; gg < HMAX; gg++) {
                        const float t = tk[h * HMAX + gg];
#pragma unroll
                        for (int i = 0; i < 4; i++) v[i] = fmaf(t, raw[gg][i], v[i]);
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; i++) s[h][i] = see[i] ? v[i] : -INFINITY;
            }
        } else {
#pragma unroll
            for (int h = 0; h < HMAX; h++) s[h] = (f32x4_t){-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        }
        // ---- 2. the block's largest score a (head, row), through LDS
#pragma unroll
        for (int h = 0; h < HMAX; h++) {
            if (h < H) {
                float v = fmaxf(fmaxf(s[h][0], s[h][1]), fmaxf(s[h][2], s[h][3]));
                v = fmaxf(v, __shfl_xor(v, 16, kWave));
                v = fmaxf(v, __shfl_xor(v, 32, kWave));
                if (g == 0) mx[wave][h][c] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < HMAX; h++) {
            if (h < H) {
                const float blk = fmaxf(fmaxf(mx[0][h][c], mx[1][h][c]), fmaxf(mx[2][h][c], mx[3][h][c]));
                const float m_new = fmaxf(m_run[h], blk);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;      // a row that has seen no key yet
                const float alpha = __expf(m_run[h] - m_safe);
                m_run[h] = m_new;
                float sum = 0.f;
                bf16x4_t w4;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e = __expf(s[h][i] - m_safe);
                    sum += e;
                    w4[i] = (bf16_t)e;
                }
                l_part[h] = l_part[h] * alpha + sum;
                *(bf16x4_t *)&ps[h][wave][c][4 * g] = w4;
                if (wave == 0 && g == 0) al[h][c] = alpha;
            }
        }
        __syncthreads();
        // ---- 3. outputs: this wave's (head, 16 value lanes) units
#pragma unroll
        for (int j = 0; j < UMAX; j++) {
            const int u = wave + 4 * j;
            if (u < units) {
                const int h = u / DVT, t = u - h * DVT, kvh = h / group;
                const float alpha = al[h][c];
                f32x4_t acc = o[j];
#pragma unroll
                for (int i = 0; i < 4; i++) acc[i] *= alpha;
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    if (kb + 32 * s2 > plast) continue;      // uniform: no key of this half is seen
                    bf16x8_t pf, vf;
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        const bf16x4_t w4 = *(const bf16x4_t *)&ps[h][2 * s2 + half][c][4 * g];
                        const int key4 = kb + 32 * s2 + 16 * half + 4 * g;
                        bf16x4_t v4 = {0, 0, 0, 0};
                        if (key4 <= plast) {
                            const int page = tbl[key4 / PS], off = key4 % PS;
                            v4 = *(const bf16x4_t *)(p.v_pages + (((size_t)page * G + kvh) * DV + 16 * t + c) * PS + off);
                        }
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            pf[4 * half + e] = w4[e];
                            vf[4 * half + e] = key4 + e <= plast ? v4[e] : (bf16_t)0.f;   // slots past the last token hold anything
                        }
                    }
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc, 0, 0, 0);
                }
                o[j] = acc;
            }
        }
        __syncthreads();   // ps, mx and al are rewritten by the next block
    }
    // the rows' sums: lanes of one row, then the four waves
#pragma unroll
    for (int h = 0; h < HMAX; h++) {
        if (h < H) {
            float v = l_part[h];
            v += __shfl_xor(v, 16, kWave);
            v += __shfl_xor(v, 32, kWave);
            if (g == 0) mx[wave][h][c] = v;
        }
    }
    __syncthreads();
    if (c >= nrows) return;
#pragma unroll
    for (int j = 0; j < UMAX; j++) {
        const int u = wave + 4 * j;
        if (u < units) {
            const int h = u / DVT, t = u - h * DVT;
            const float l = (mx[0][h][c] + mx[1][h][c]) + (mx[2][h][c] + mx[3][h][c]);
            float f = l > 0.f ? 1.0f / l : 0.f;
            if (p.gate != nullptr) f *= 1.0f / (1.0f + __expf(-(float)p.gate[(size_t)(first + c) * p.gate_stride + h]));
            bf16x4_t r4;
#pragma unroll
            for (int i = 0; i < 4; i++) r4[i] = (bf16_t)(o[j][i] * f);
            *(bf16x4_t *)(p.out + (size_t)(first + c) * out_row + (size_t)h * DV + 16 * t + 4 * g) = r4;
        }
    }
}

template <int HMAX>
int launch_tiles(const TalkArgs &a, int tiles, size_t lds, hipStream_t stream) {
    constexpr int KSMAX = 8, UMAX = HMAX * 8 / 4;
    auto kernel = talking_tile_kernel<HMAX, KSMAX, UMAX>;
    // the kernel's own arrays (mixing matrix, maxima, factors, weights) come on top of the queries: beyond the default
    // 64 KiB of both together the larger amount has to be asked for
    constexpr size_t own = sizeof(float) * (HMAX * HMAX + 5 * HMAX * kTileRows) + sizeof(bf16_t) * HMAX * 4 * kTileRows * 16;
    FLLM_REQUIRE(own + lds <= 160 * 1024, "talking_attention: %zu bytes of LDS", own + lds);
    if (own + lds > 60 * 1024)
        FLLM_REQUIRE(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,
                     "talking_attention: cannot have %zu bytes of LDS", lds);
    hipLaunchKernelGGL(kernel, dim3(tiles), dim3(kThreads), lds, stream, a);
    return fllm_check_launch("talking_attention (matrix cores)");
}

}  // namespace

// 1: the shape is not taken, the caller runs the plain kernel
int fllm_talking_attention_bf16_fast(const void *q, const void *gate, int gate_stride, const void *k_pages, const void *v_pages,
                                     const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                                     const int32_t *seg_start, int num_segs, const float *talk, const float *temp, void *out,
                                     int rows, int heads, int kv_heads, int k_dim, int v_dim, int page_size, float scale, int chunk,
                                     int key_chunk, int max_context, hipStream_t stream) {
    (void)max_context;
    if (key_chunk != 8 || k_dim % 32 != 0 || k_dim > 256 || v_dim % 16 != 0 || v_dim > 128 || heads > 16 || page_size % 4 != 0)
        return 1;
    const size_t lds = (size_t)kTileRows * (heads * k_dim + 8) * sizeof(bf16_t);
    if (lds > 96 * 1024) return 1;      // wider rows of queries go to the plain kernel
    if (((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15) return 1;
    TalkArgs a;
    a.q = (const bf16_t *)q;
    a.gate = (const bf16_t *)gate;
    a.gate_stride = gate_stride;
    a.k_pages = (const bf16_t *)k_pages;
    a.v_pages = (const bf16_t *)v_pages;
    a.tables = tables;
    a.table_stride = table_stride;
    a.row_pos = row_pos;
    a.row_seg = row_seg;
    a.seg_start = seg_start;
    a.num_segs = num_segs;
    a.talk = talk;
    a.temp = temp;
    a.out = (bf16_t *)out;
    a.rows = rows;
    a.heads = heads;
    a.kv_heads = kv_heads;
    a.k_dim = k_dim;
    a.v_dim = v_dim;
    a.page_size = page_size;
    a.scale = scale;
    a.chunk = chunk;
    // every segment's rows in tiles of 16: at most rows / 16 full tiles and one ragged tile a segment
    const int tiles = rows / kTileRows + num_segs;
    return heads <= 8 ? launch_tiles<8>(a, tiles, lds, stream) : launch_tiles<16>(a, tiles, lds, stream);
}
