// Matrix-core form of the attention whose heads talk to each other (talking_attention.hip says what is computed),
// bfloat16 operands, float32 scores, statistics and sums.
//
// A workgroup of four waves takes 16 consecutive rows of one request (a prompt portion's row tile, or a decode step's
// single row) with ALL heads, because a mixed score needs every head's raw score of the same (row, key).  It walks the
// keys the tile sees in blocks of 64; with `splits` > 1 the blocks of a tile are dealt out to that many workgroups,
// which leave their running maxima, sums and unnormalised outputs in a workspace that a second kernel merges (few row
// tiles would otherwise leave most of the 256 compute units idle: a decode step has one tile a request).
//
// Keys and values pass through LDS, one key/value head at a time (a "stage": 64 keys x k_dim, then 64 keys x v_dim):
// all threads load the stage after the next one into registers while the waves multiply from the stage in LDS, so the
// latency of the pages is hidden behind the products and LDS holds one head's block however many heads there are.
// The products are the transposed ones, v_mfma_f32_16x16x32_bf16 with D[m = 4 (l / 16) + i][n = l % 16], so that a
// lane keeps one row throughout:
//
//   1. wave w takes the block's keys 16 w .. 16 w + 15: for every head  raw_g^T[key][row] = K_{g / group} Q_g^T
//      (A = 16 keys x 32 lanes from the stage, B = the rows' queries from LDS).  A lane then holds, for its four
//      (key, row) pairs, the raw scores of all heads: the mix  s_h = sum_g talk'[h, g] raw_g  is lane-local
//      (talk'[h, g] = talk[h, g] * scale * temp[g], prepared in LDS once).
//   2. the block's largest score a (head, row) goes through LDS (four waves hold different keys); every wave computes
//      the same running maximum, weighs its scores, keeps its share of the running sum and leaves the weights in LDS
//      as bfloat16, [head][key group][row][16 keys].
//   3. the outputs  O_h^T[lane of v][row] += V_{h / group}^T P_h^T: wave w owns the value lanes 16 w .. 16 w + 15 and
//      64 + 16 w .. of every head, so a value fragment (A) is read once a key/value head and serves its whole group;
//      B = weights from LDS.  The k slots of this product hold the keys 4 g + i of two key groups, the order step 2
//      left them in.
//
// Rows of a tile see different key ranges when a chunk of positions ends inside the tile: the mask is per (row, key).
#include "api.h"
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kTileRows = 16;
constexpr int kKeyBlock = 64;
constexpr int kVPitch = kKeyBlock + 4;      // a value lane's 64 keys in the stage, padded

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
    int splits;
    float *ws;       // splits > 1: [tile][split] { m [heads][16], l [heads][16], o [16][heads][v_dim] }
};

__device__ __forceinline__ size_t part_floats(int heads, int v_dim) { return (size_t)kTileRows * heads * (2 + v_dim); }

// which rows: the workgroup's tile among the tiles of all segments
__device__ __forceinline__ bool find_tile(const TalkArgs &p, int tile, int &seg, int &first, int &nrows) {
    int before = 0;
    for (int s = 0; s < p.num_segs; s++) {
        const int r0 = p.seg_start[s], n = p.seg_start[s + 1] - r0;
        const int tiles = (n + kTileRows - 1) / kTileRows;
        if (tile < before + tiles) {
            const int t = tile - before;
            seg = s;
            first = r0 + t * kTileRows;
            nrows = n - t * kTileRows < kTileRows ? n - t * kTileRows : kTileRows;
            return true;
        }
        before += tiles;
    }
    return false;
}

template <int HMAX>
__global__ void __launch_bounds__(kThreads)
talking_tile_kernel(const TalkArgs p) {
    constexpr int KSMAX = 8;       // k_dim <= 256
    constexpr int TS = 2;          // v_dim <= 128: two 16-lane pieces a wave
    constexpr int PRE = 8;         // 16-byte registers a thread holds of the stage in flight
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    __shared__ float tk[HMAX * HMAX];
    __shared__ float mx[4][HMAX][kTileRows];
    __shared__ float al[HMAX][kTileRows];
    __shared__ __attribute__((aligned(16))) bf16_t ps[HMAX][4][kTileRows][16];

    const int H = p.heads, G = p.kv_heads, D = p.k_dim, DV = p.v_dim, PS = p.page_size;
    const int group = H / G, KS = D / 32, DVT = DV / 16;
    const int QP = H * D + 8, KP = D + 8;
    bf16_t *qs = (bf16_t *)lds_raw;
    bf16_t *stage = qs + kTileRows * QP;
    int seg, first, nrows;
    if (!find_tile(p, blockIdx.x, seg, first, nrows)) return;
    const int S = p.splits, split = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const size_t out_row = (size_t)H * DV;
    if (p.row_seg[first] < 0) {   // padding rows of a captured step
        if (split == 0)
            for (int i = tid; i < nrows * H * DV; i += kThreads) p.out[(size_t)first * out_row + i] = (bf16_t)0.f;
        return;
    }
    const int pos0 = p.row_pos[first], plast = pos0 + nrows - 1;
    const int lo_tile = p.chunk > 0 ? pos0 - pos0 % p.chunk : 0;
    const int kb_start = lo_tile & ~15;
    const int32_t *tbl = p.tables + (size_t)seg * p.table_stride;
    const int pos_c = c < nrows ? pos0 + c : -1;
    const int lo_c = p.chunk > 0 && pos_c >= 0 ? pos_c - pos_c % p.chunk : 0;
    const int nblk = (plast - kb_start) / kKeyBlock + 1;
    const int my_blocks = split < nblk ? (nblk - split + S - 1) / S : 0;
    const int total_stages = my_blocks * 2 * G;

    // a stage: block b of this workgroup's blocks, then K of key/value head 0 .. G - 1, then V of 0 .. G - 1
    bf16x8_t pre[PRE];
    auto load_stage = [&](int si) {
        const int b = si / (2 * G), st = si - b * 2 * G;
        const int kb = kb_start + kKeyBlock * (split + S * b);
        if (st < G) {
            const int key = kb + (tid & 63);
            const int key_a = key <= plast ? key : plast;      // clamped: masked later
            const int page = tbl[key_a / PS], off = key_a % PS;
#pragma unroll
            for (int r = 0; r < PRE; r++) {
                const int j = (tid >> 6) + 4 * r;      // which 8 lanes of the key
                if (8 * j < D) pre[r] = *(const bf16x8_t *)(p.k_pages + key_offset(page, G, st, PS, D, off, 8 * j));
            }
        } else {
            const int kvh = st - G;
            const int key4 = kb + (tid & 15) * 4;
            const bool any = key4 <= plast;
            int page = 0, off = 0;
            if (any) { page = tbl[key4 / PS]; off = key4 % PS; }
#pragma unroll
            for (int r = 0; r < PRE; r++) {
                const int dv = (tid >> 4) + 16 * r;
                if (dv < DV) {
                    bf16x4_t v4 = {0, 0, 0, 0};
                    if (any) v4 = *(const bf16x4_t *)(p.v_pages + (((size_t)page * G + kvh) * DV + dv) * PS + off);
#pragma unroll
                    for (int e = 0; e < 4; e++) pre[r][e] = key4 + e <= plast ? v4[e] : (bf16_t)0.f;   // slots past the last token hold anything
                }
            }
        }
    };
    auto store_stage = [&](int si) {
        const int st = si % (2 * G);
        if (st < G) {
#pragma unroll
            for (int r = 0; r < PRE; r++) {
                const int j = (tid >> 6) + 4 * r;
                if (8 * j < D) *(bf16x8_t *)(stage + (tid & 63) * KP + 8 * j) = pre[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < PRE; r++) {
                const int dv = (tid >> 4) + 16 * r;
                if (dv < DV) {
                    bf16x4_t v4;
#pragma unroll
                    for (int e = 0; e < 4; e++) v4[e] = pre[r][e];
                    *(bf16x4_t *)(stage + dv * kVPitch + (tid & 15) * 4) = v4;
                }
            }
        }
    };
    if (total_stages > 0) load_stage(0);

    // queries of the tile and the mixing matrix into LDS
    {
        const int per_row = H * D / 8;
        for (int i = tid; i < kTileRows * per_row; i += kThreads) {
            const int r = i / per_row, e = (i - r * per_row) * 8;
            bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (r < nrows) v = *(const bf16x8_t *)(p.q + (size_t)(first + r) * H * D + e);
            *(bf16x8_t *)(qs + r * QP + e) = v;
        }
        for (int i = tid; i < HMAX * HMAX; i += kThreads) {
            const int h = i / HMAX, gg = i % HMAX;
            tk[i] = h < H && gg < H ? p.talk[h * H + gg] * (p.scale * p.temp[gg]) : 0.f;
        }
    }
    if (total_stages > 0) store_stage(0);
    __syncthreads();
    if (total_stages > 1) load_stage(1);

    float m_run[HMAX], l_part[HMAX];
    f32x4_t o[HMAX][TS];
#pragma unroll
    for (int h = 0; h < HMAX; h++) {
        m_run[h] = -INFINITY;
        l_part[h] = 0.f;
#pragma unroll
        for (int ts = 0; ts < TS; ts++) o[h][ts] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    }

    int si = 0;      // the stage that lies in LDS; the one after it is in flight in `pre`
    auto next_stage = [&]() {
        __syncthreads();                      // every wave is done with the stage in LDS
        if (si + 1 < total_stages) store_stage(si + 1);
        __syncthreads();
        si++;
        if (si + 1 < total_stages) load_stage(si + 1);
    };

    for (int b = 0; b < my_blocks; b++) {
        const int kb = kb_start + kKeyBlock * (split + S * b);
        // ---- 1. raw scores of this wave's 16 keys for every head, one key/value head a stage, then the mix
        const int key0 = kb + 16 * wave;
        const bool active = key0 <= plast;      // wave-uniform
        f32x4_t raw[HMAX];
#pragma unroll
        for (int h = 0; h < HMAX; h++) raw[h] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        for (int kvh = 0; kvh < G; kvh++) {
            if (active) {
                bf16x8_t kf[KSMAX];
#pragma unroll
                for (int ks = 0; ks < KSMAX; ks++)
                    if (ks < KS) kf[ks] = *(const bf16x8_t *)(stage + (16 * wave + c) * KP + 32 * ks + 8 * g);
                const int h_lo = kvh * group, h_hi = h_lo + group;
#pragma unroll
                for (int h = 0; h < HMAX; h++) {
                    if (h >= h_lo && h < h_hi) {
#pragma unroll
                        for (int ks = 0; ks < KSMAX; ks++)
                            if (ks < KS) {
                                const bf16x8_t qf = *(const bf16x8_t *)(qs + c * QP + h * D + 32 * ks + 8 * g);
                                raw[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf, raw[h], 0, 0, 0);
                            }
                    }
                }
            }
            next_stage();
        }
        f32x4_t s[HMAX];
        if (active) {
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
        // ---- 3. outputs, one key/value head a stage: this wave's value lanes of every head of the group
        for (int kvh = 0; kvh < G; kvh++) {
            const int h_lo = kvh * group, h_hi = h_lo + group;
#pragma unroll
            for (int ts = 0; ts < TS; ts++) {
                const int t = wave + 4 * ts;
                if (t < DVT) {
                    bf16x8_t vf[2];
#pragma unroll
                    for (int s2 = 0; s2 < 2; s2++) {
                        const bf16x4_t a4 = *(const bf16x4_t *)(stage + (16 * t + c) * kVPitch + 32 * s2 + 4 * g);
                        const bf16x4_t b4 = *(const bf16x4_t *)(stage + (16 * t + c) * kVPitch + 32 * s2 + 16 + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; e++) { vf[s2][e] = a4[e]; vf[s2][4 + e] = b4[e]; }
                    }
#pragma unroll
                    for (int h = 0; h < HMAX; h++) {
                        if (h >= h_lo && h < h_hi) {
                            const float alpha = al[h][c];
                            f32x4_t acc = o[h][ts];
#pragma unroll
                            for (int i = 0; i < 4; i++) acc[i] *= alpha;
#pragma unroll
                            for (int s2 = 0; s2 < 2; s2++) {
                                if (kb + 32 * s2 > plast) continue;      // uniform: no key of this half is seen
                                const bf16x4_t a4 = *(const bf16x4_t *)&ps[h][2 * s2][c][4 * g];
                                const bf16x4_t b4 = *(const bf16x4_t *)&ps[h][2 * s2 + 1][c][4 * g];
                                bf16x8_t pf;
#pragma unroll
                                for (int e = 0; e < 4; e++) { pf[e] = a4[e]; pf[4 + e] = b4[e]; }
                                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[s2], pf, acc, 0, 0, 0);
                            }
                            o[h][ts] = acc;
                        }
                    }
                }
            }
            next_stage();      // its barriers also keep ps, mx and al from the next block's writes
        }
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
    if (S > 1) {
        // this workgroup's share of the tile: maxima and sums [heads][16], unnormalised outputs [16][heads][v_dim]
        float *part = p.ws + ((size_t)blockIdx.x * S + split) * part_floats(H, DV);
        float *part_o = part + 2 * kTileRows * H;
#pragma unroll
        for (int h = 0; h < HMAX; h++) {
            if (h < H) {
                if (wave == 0 && g == 0) {
                    part[h * kTileRows + c] = m_run[h];
                    part[(H + h) * kTileRows + c] = (mx[0][h][c] + mx[1][h][c]) + (mx[2][h][c] + mx[3][h][c]);
                }
#pragma unroll
                for (int ts = 0; ts < TS; ts++) {
                    const int t = wave + 4 * ts;
                    if (t < DVT) *(f32x4_t *)(part_o + ((size_t)c * H + h) * DV + 16 * t + 4 * g) = o[h][ts];
                }
            }
        }
        return;
    }
    if (c >= nrows) return;
#pragma unroll
    for (int h = 0; h < HMAX; h++) {
        if (h < H) {
            const float l = (mx[0][h][c] + mx[1][h][c]) + (mx[2][h][c] + mx[3][h][c]);
            float f = l > 0.f ? 1.0f / l : 0.f;
            if (p.gate != nullptr) f *= 1.0f / (1.0f + __expf(-(float)p.gate[(size_t)(first + c) * p.gate_stride + h]));
#pragma unroll
            for (int ts = 0; ts < TS; ts++) {
                const int t = wave + 4 * ts;
                if (t < DVT) {
                    bf16x4_t r4;
#pragma unroll
                    for (int i = 0; i < 4; i++) r4[i] = (bf16_t)(o[h][ts][i] * f);
                    *(bf16x4_t *)(p.out + (size_t)(first + c) * out_row + (size_t)h * DV + 16 * t + 4 * g) = r4;
                }
            }
        }
    }
}

// The shares of a tile's workgroups into the rows' outputs: out = sum_s o_s e^(m_s - m) / sum_s l_s e^(m_s - m) * gate.
__global__ void __launch_bounds__(kThreads) talking_merge_kernel(const TalkArgs p) {
    int seg, first, nrows;
    if (!find_tile(p, blockIdx.x, seg, first, nrows)) return;
    if (p.row_seg[first] < 0) return;      // padding rows: the tile kernel has written zeros
    const int H = p.heads, DV = p.v_dim, S = p.splits;
    const size_t per = part_floats(H, DV);
    const float *parts = p.ws + (size_t)blockIdx.x * S * per;
    const int quads = DV / 4;
    for (int i = threadIdx.x; i < nrows * H * quads; i += kThreads) {
        const int c = i / (H * quads), rem = i - c * H * quads, h = rem / quads, d4 = (rem - h * quads) * 4;
        float m = -INFINITY;
        for (int s = 0; s < S; s++) m = fmaxf(m, parts[s * per + h * kTileRows + c]);
        float l = 0.f;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (m > -INFINITY) {
            for (int s = 0; s < S; s++) {
                const float *part = parts + s * per;
                const float w = __expf(part[h * kTileRows + c] - m);
                l += part[(H + h) * kTileRows + c] * w;
                const f32x4_t o4 = *(const f32x4_t *)(part + 2 * kTileRows * H + ((size_t)c * H + h) * DV + d4);
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] = fmaf(o4[e], w, acc[e]);
            }
        }
        float f = l > 0.f ? 1.0f / l : 0.f;
        if (p.gate != nullptr) f *= 1.0f / (1.0f + __expf(-(float)p.gate[(size_t)(first + c) * p.gate_stride + h]));
        bf16x4_t r4;
#pragma unroll
        for (int e = 0; e < 4; e++) r4[e] = (bf16_t)(acc[e] * f);
        *(bf16x4_t *)(p.out + (size_t)(first + c) * H * DV + (size_t)h * DV + d4) = r4;
    }
}

template <int HMAX>
int launch_tiles(const TalkArgs &a, int tiles, size_t lds, hipStream_t stream) {
    auto kernel = talking_tile_kernel<HMAX>;
    // the kernel's own arrays (mixing matrix, maxima, factors, weights) come on top of the queries and the stage: beyond
    // the default 64 KiB of both together the larger amount has to be asked for
    constexpr size_t own = sizeof(float) * (HMAX * HMAX + 5 * HMAX * kTileRows) + sizeof(bf16_t) * HMAX * 4 * kTileRows * 16;
    if (own + lds > 160 * 1024) return 1;
    if (own + lds > 60 * 1024) {
        static bool asked = false;
        if (!asked) {
            FLLM_REQUIRE(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - (int)own) ==
                             hipSuccess, "talking_attention: cannot have %zu bytes of LDS", own + lds);
            asked = true;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(tiles, a.splits), dim3(kThreads), lds, stream, a);
    int rc = fllm_check_launch("talking_attention (matrix cores)");
    if (rc == 0 && a.splits > 1) {
        hipLaunchKernelGGL(talking_merge_kernel, dim3(tiles), dim3(kThreads), 0, stream, a);
        rc = fllm_check_launch("talking_attention (merge)");
    }
    return rc;
}

}  // namespace

// Floats of workspace that `splits` workgroups a tile need for `rows` rows in `num_segs` segments.
extern "C" size_t fllm_talking_attention_workspace(int rows, int num_segs, int heads, int v_dim, int splits) {
    if (splits <= 1) return 0;
    return (size_t)(rows / kTileRows + num_segs) * splits * kTileRows * heads * (2 + v_dim);
}

// 1: the shape is not taken, the caller runs the plain kernel
int fllm_talking_attention_bf16_fast(const void *q, const void *gate, int gate_stride, const void *k_pages, const void *v_pages,
                                     const int32_t *tables, int table_stride, const int32_t *row_pos, const int32_t *row_seg,
                                     const int32_t *seg_start, int num_segs, const float *talk, const float *temp, void *out,
                                     int rows, int heads, int kv_heads, int k_dim, int v_dim, int page_size, float scale, int chunk,
                                     int key_chunk, int max_context, int splits, float *ws, size_t ws_floats, hipStream_t stream) {
    (void)max_context;
    if (key_chunk != 8 || k_dim % 32 != 0 || k_dim > 256 || v_dim % 16 != 0 || v_dim > 128 || heads > 16 || page_size % 4 != 0)
        return 1;
    const size_t stage = (size_t)kKeyBlock * (k_dim + 8) > (size_t)v_dim * kVPitch ? (size_t)kKeyBlock * (k_dim + 8) : (size_t)v_dim * kVPitch;
    const size_t lds = ((size_t)kTileRows * (heads * k_dim + 8) + stage) * sizeof(bf16_t);
    if (((uintptr_t)q | (uintptr_t)out | (uintptr_t)k_pages | (uintptr_t)v_pages) & 15) return 1;
    if (splits < 1) splits = 1;
    if (splits > 1) {
        FLLM_REQUIRE(ws != nullptr && ((uintptr_t)ws & 15) == 0 &&
                         ws_floats >= fllm_talking_attention_workspace(rows, num_segs, heads, v_dim, splits),
                     "talking_attention: %d workgroups a tile need a workspace of %zu floats, aligned to 16 bytes (%zu given)", splits,
                     fllm_talking_attention_workspace(rows, num_segs, heads, v_dim, splits), ws_floats);
    }
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
    a.splits = splits;
    a.ws = ws;
    // every segment's rows in tiles of 16: at most rows / 16 full tiles and one ragged tile a segment
    const int tiles = rows / kTileRows + num_segs;
    return heads <= 8 ? launch_tiles<8>(a, tiles, lds, stream) : launch_tiles<16>(a, tiles, lds, stream);
}
