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
    int gs;          // key/value heads a stage holds
    int ptab;        // page numbers of a tile's keys that fit into LDS (0: they are read from the table in memory)
};

__device__ __forceinline__ size_t part_floats(int heads, int v_dim) { return (size_t)kTileRows * heads * (2 + v_dim); }

// which rows: the workgroup's tile among the tiles of all segments.  The segments' first rows come through LDS in one
// load where they fit (`starts`, kMaxSegsLds + 1 ints): a scan over memory would wait for every segment in turn.
constexpr int kMaxSegsLds = 255;

__device__ __forceinline__ bool find_tile(const TalkArgs &p, int tile, int *starts, int &seg, int &first, int &nrows) {
    const bool in_lds = p.num_segs <= kMaxSegsLds;
    if (in_lds) {
        if ((int)threadIdx.x <= p.num_segs) starts[threadIdx.x] = p.seg_start[threadIdx.x];
        __syncthreads();
    }
    int before = 0;
    for (int s = 0; s < p.num_segs; s++) {
        const int r0 = in_lds ? starts[s] : p.seg_start[s], n = (in_lds ? starts[s + 1] : p.seg_start[s + 1]) - r0;
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
    const int GS = p.gs, NST = (G + GS - 1) / GS;      // key/value heads a stage, stages of keys (and of values) a block
    const int QP = H * D + 8, KP = GS * D + 8;
    bf16_t *qs = (bf16_t *)lds_raw;
    bf16_t *stage = qs + kTileRows * QP;
    const size_t stage_elems = (size_t)kKeyBlock * KP > (size_t)GS * DV * kVPitch ? (size_t)kKeyBlock * KP : (size_t)GS * DV * kVPitch;
    int *ptab = (int *)(stage + ((stage_elems + 7) & ~(size_t)7));
    __shared__ int starts[kMaxSegsLds + 1];
    int seg, first, nrows;
    // the last tiles of a prompt see the most keys: they start first, so that the short ones fill the gaps at the end
    const int tile = gridDim.x - 1 - blockIdx.x;
    if (!find_tile(p, tile, starts, seg, first, nrows)) return;
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
    const int total_stages = my_blocks * 2 * NST;
    // the pages of the tile's keys: through LDS in one load where they fit, so that a stage's loads wait for no lookup
    const int page0 = kb_start / PS, npages = plast / PS - page0 + 1;
    const bool pages_in_lds = npages <= p.ptab;
    if (pages_in_lds)
        for (int i = tid; i < npages; i += kThreads) ptab[i] = tbl[page0 + i];
    auto page_of = [&](int key) __attribute__((always_inline)) { return pages_in_lds ? ptab[key / PS - page0] : tbl[key / PS]; };

    // a stage: block b of this workgroup's blocks, then K of the key/value heads GS at a time, then V likewise
    bf16x8_t pre[PRE];
    auto load_stage = [&](int si) __attribute__((always_inline)) {
        const int b = si / (2 * NST), st = si - b * 2 * NST;
        const int kb = kb_start + kKeyBlock * (split + S * b);
        if (st < NST) {
            const int kvh0 = st * GS;
            const int key = kb + (tid & 63);
            const int key_a = key <= plast ? key : plast;      // clamped: masked later
            const int page = page_of(key_a), off = key_a % PS;
            const int per_head = D >> 3;                       // at least 4: a step of 4 wraps once at most
            int l = 0, j = tid >> 6;                           // which head of the stage, which 8 lanes of its keys
#pragma unroll
            for (int r = 0; r < PRE; r++) {
                if (l < GS && kvh0 + l < G) pre[r] = *(const bf16x8_t *)(p.k_pages + key_offset(page, G, kvh0 + l, PS, D, off, 8 * j));
                j += 4;
                if (j >= per_head) { j -= per_head; l++; }
            }
        } else {
            const int kvh0 = (st - NST) * GS;
            const int key4 = kb + (tid & 15) * 4;
            const bool any = key4 <= plast;
            int page = 0, off = 0;
            if (any) { page = page_of(key4); off = key4 % PS; }
            int l = 0, dv = tid >> 4;                          // which head of the stage, which of its value lanes
#pragma unroll
            for (int r = 0; r < 2 * PRE; r++) {
                if (l < GS && kvh0 + l < G) {
                    bf16x4_t v4 = {0, 0, 0, 0};
                    if (any) v4 = *(const bf16x4_t *)(p.v_pages + (((size_t)page * G + kvh0 + l) * DV + dv) * PS + off);
#pragma unroll
                    for (int e = 0; e < 4; e++) pre[r >> 1][4 * (r & 1) + e] = key4 + e <= plast ? v4[e] : (bf16_t)0.f;   // slots past the last token hold anything
                }
                dv += 16;
                if (dv >= DV) { dv -= DV; l++; }               // v_dim is a multiple of 16
            }
        }
    };
    auto store_stage = [&](int si) __attribute__((always_inline)) {
        const int st = si % (2 * NST);
        if (st < NST) {
#pragma unroll
            for (int r = 0; r < PRE; r++) {
                const int jj = (tid >> 6) + 4 * r;
                if (8 * jj < GS * D) *(bf16x8_t *)(stage + (tid & 63) * KP + 8 * jj) = pre[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < 2 * PRE; r++) {
                const int row = (tid >> 4) + 16 * r;
                if (row < GS * DV) {
                    bf16x4_t v4;
#pragma unroll
                    for (int e = 0; e < 4; e++) v4[e] = pre[r >> 1][4 * (r & 1) + e];
                    *(bf16x4_t *)(stage + row * kVPitch + (tid & 15) * 4) = v4;
                }
            }
        }
    };
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
    __syncthreads();

    float m_run[HMAX], l_part[HMAX];
    f32x4_t o[HMAX][TS];
#pragma unroll
    for (int h = 0; h < HMAX; h++) {
        m_run[h] = -INFINITY;
        l_part[h] = 0.f;
#pragma unroll
        for (int ts = 0; ts < TS; ts++) o[h][ts] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    }

    // One loop over the stages, with one place each where a stage is loaded and stored (the kernel's code has to stay
    // within the instruction cache): pass -2 loads stage 0, pass -1 stores it and loads stage 1, pass si >= 0 multiplies
    // from stage si in LDS while stage si + 1 is in flight in `pre`.
    f32x4_t raw[HMAX];
    for (int si = -2; si < total_stages; si++) {
        if (si >= 0) {
            const int b = si / (2 * NST), st = si - b * 2 * NST;
            const int kb = kb_start + kKeyBlock * (split + S * b);
            const int key0 = kb + 16 * wave;
            const bool active = key0 <= plast;      // wave-uniform
            if (st < NST) {
                // ---- 1. raw scores of this wave's 16 keys for the heads of the stage's key/value heads
                if (st == 0) {
#pragma unroll
                    for (int h = 0; h < HMAX; h++) raw[h] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                }
                if (active) {
                    for (int l = 0; l < GS && st * GS + l < G; l++) {
                        bf16x8_t kf[KSMAX];
#pragma unroll
                        for (int ks = 0; ks < KSMAX; ks++)
                            if (ks < KS) kf[ks] = *(const bf16x8_t *)(stage + (16 * wave + c) * KP + l * D + 32 * ks + 8 * g);
                        const int h_lo = (st * GS + l) * group, h_hi = h_lo + group;
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
                }
                if (st == NST - 1) {
                    // ---- the mix, lane-local
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
                    // the barrier below, before the next stage is stored, also publishes ps and al
                }
            } else {
                // ---- 3. outputs: this wave's value lanes of every head of the stage's key/value heads
                for (int l = 0; l < GS && (st - NST) * GS + l < G; l++) {
                    const int h_lo = ((st - NST) * GS + l) * group, h_hi = h_lo + group;
                    const int lrow = l * DV;
#pragma unroll
                    for (int ts = 0; ts < TS; ts++) {
                        const int t = wave + 4 * ts;
                        if (t < DVT) {
                            bf16x8_t vf[2];
#pragma unroll
                            for (int s2 = 0; s2 < 2; s2++) {
                                const bf16x4_t a4 = *(const bf16x4_t *)(stage + (lrow + 16 * t + c) * kVPitch + 32 * s2 + 4 * g);
                                const bf16x4_t b4 = *(const bf16x4_t *)(stage + (lrow + 16 * t + c) * kVPitch + 32 * s2 + 16 + 4 * g);
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
                }
            }
        }
        __syncthreads();                      // every wave is done with the stage in LDS (and ps, mx, al of its block)
        if (si + 1 >= 0 && si + 1 < total_stages) store_stage(si + 1);
        __syncthreads();
        if (si + 2 < total_stages) load_stage(si + 2);
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
        float *part = p.ws + ((size_t)tile * S + split) * part_floats(H, DV);
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

// The shares of a tile's workgroups into the rows' outputs, a workgroup a (tile, head): out = sum_s o_s e^(m_s - m) / sum_s l_s e^(m_s - m) * gate.
__global__ void __launch_bounds__(kThreads) talking_merge_kernel(const TalkArgs p) {
    __shared__ int starts[kMaxSegsLds + 1];
    int seg, first, nrows;
    if (!find_tile(p, blockIdx.x, starts, seg, first, nrows)) return;
    if (p.row_seg[first] < 0) return;      // padding rows: the tile kernel has written zeros
    const int H = p.heads, DV = p.v_dim, S = p.splits, h = blockIdx.y;
    const size_t per = part_floats(H, DV);
    const float *parts = p.ws + (size_t)blockIdx.x * S * per;
    const int quads = DV / 4;
    for (int i = threadIdx.x; i < nrows * quads; i += kThreads) {
        const int c = i / quads, d4 = (i - c * quads) * 4;
        float m = -INFINITY;
#pragma unroll 4
        for (int s = 0; s < S; s++) m = fmaxf(m, parts[s * per + h * kTileRows + c]);
        float l = 0.f;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (m > -INFINITY) {
#pragma unroll 4
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

// ---- decode steps: one row a request -----------------------------------------------------------------------------------
// With a single row the 16 columns of a product are the HEADS that share a key/value head (the same position's queries),
// not 16 positions: one chain of products gives a block's raw scores of a whole group, and a lane keeps a few numbers, so
// many waves fit a compute unit and hide one another's waits.  A workgroup takes one request's row and walks its key
// blocks of 64 (or its share of them, `splits` as above):
//   1. wave w, keys 16 w .. 16 w + 15 straight from the pages: raw^T[key][head of the group] = K Q^T a key/value head;
//      the raw scores go to LDS as [key][head].
//   2. lane = key, wave w owns the heads w, w + 4, ..: the mix over a key's raw scores, then maximum, weights and sums of
//      a head's 64 keys inside one wave; the weights go to LDS as bfloat16 [head column][key].
//   3. wave w, value lanes 16 w .. and 64 + 16 w ..: O^T[value lane][head of the group] += V^T P^T a key/value head.
constexpr int kDecGMax = 8;        // key/value heads
constexpr int kDecPPitch = kKeyBlock + 8;

__device__ __forceinline__ float wave_max64(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

__device__ __forceinline__ size_t decode_part_floats(int heads, int v_dim) { return (size_t)heads * (2 + v_dim); }

template <int HW>      // heads a wave owns in step 2: at most 4 HW heads
__global__ void __launch_bounds__(kThreads)
talking_decode_kernel(const TalkArgs p) {
    constexpr int KSMAX = 8, TS = 2;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int H = p.heads, G = p.kv_heads, D = p.k_dim, DV = p.v_dim, PS = p.page_size;
    const int group = H / G, KS = D / 32, DVT = DV / 16, HP = H | 1;
    float *tk = (float *)lds_raw;                       // [H][H]
    float *rawl = tk + H * H;                           // [64 keys][HP]
    float *alv = rawl + kKeyBlock * HP;                 // [H] factors of this block
    float *mlv = alv + H;                               // [2][H] maxima and sums at the end
    bf16_t *qs = (bf16_t *)(mlv + 2 * H + ((4 - ((H * H + kKeyBlock * HP + 3 * H) & 3)) & 3));      // [H][D], on 16 bytes
    bf16_t *ps2 = qs + H * D;                           // [G * 16 head columns][64 keys + 8]
    const int seg = blockIdx.x, split = blockIdx.y, S = p.splits;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int r = seg;      // every segment has one row: its first row is its own number, no lookup to wait for
    const size_t out_row = (size_t)H * DV;
    if (p.row_seg[r] < 0) {   // padding rows of a captured step
        if (split == 0)
            for (int i = tid; i < H * DV; i += kThreads) p.out[(size_t)r * out_row + i] = (bf16_t)0.f;
        return;
    }
    const int pos = p.row_pos[r];
    const int lo = p.chunk > 0 ? pos - pos % p.chunk : 0;
    const int kb_start = lo & ~15;
    const int32_t *tbl = p.tables + (size_t)seg * p.table_stride;
    const int nblk = (pos - kb_start) / kKeyBlock + 1;
    const int my_blocks = split < nblk ? (nblk - split + S - 1) / S : 0;

    for (int i = tid; i < H * D / 8; i += kThreads) *(bf16x8_t *)(qs + 8 * i) = *(const bf16x8_t *)(p.q + (size_t)r * H * D + 8 * i);
    for (int i = tid; i < H * H; i += kThreads) tk[i] = p.talk[i] * (p.scale * p.temp[i % H]);
    __syncthreads();

    float m_run[HW], l_run[HW];
#pragma unroll
    for (int j = 0; j < HW; j++) { m_run[j] = -INFINITY; l_run[j] = 0.f; }
    f32x4_t o[kDecGMax][TS];
#pragma unroll
    for (int k = 0; k < kDecGMax; k++)
#pragma unroll
        for (int ts = 0; ts < TS; ts++) o[k][ts] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    for (int b = 0; b < my_blocks; b++) {
        const int kb = kb_start + kKeyBlock * (split + S * b);
        // the pages of the keys whose values this lane takes in step 3: asked for now, so that step 3 waits for no lookup
        int vpage[2];
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) {
            const int key8 = kb + 32 * s2 + 8 * g;
            vpage[s2] = key8 <= pos ? tbl[key8 / PS] : 0;
        }
        // ---- 1. raw scores of this wave's 16 keys, a key/value head at a time
        if (kb + 16 * wave <= pos) {
            const int key = kb + 16 * wave + c;
            const int key_a = key <= pos ? key : pos;      // clamped: masked in step 2
            const int page = tbl[key_a / PS], off = key_a % PS;
            for (int kvh = 0; kvh < G; kvh++) {
                const int hq = kvh * group + c < H ? kvh * group + c : H - 1;      // columns beyond the group: any finite query
                f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KSMAX; ks++)
                    if (ks < KS) {
                        const bf16x8_t kf = *(const bf16x8_t *)(p.k_pages + key_offset(page, G, kvh, PS, D, off, 32 * ks + 8 * g));
                        const bf16x8_t qf = *(const bf16x8_t *)(qs + hq * D + 32 * ks + 8 * g);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf, acc, 0, 0, 0);
                    }
                if (c < group) {
#pragma unroll
                    for (int i = 0; i < 4; i++) rawl[(16 * wave + 4 * g + i) * HP + kvh * group + c] = acc[i];
                }
            }
        }
        __syncthreads();
        // ---- 2. lane = key: the mix of its raw scores for this wave's heads, then the heads' maxima, weights and sums
        {
            const int key = kb + lane;
            const bool see = key >= lo && key <= pos;
            float sc[HW];
#pragma unroll
            for (int j = 0; j < HW; j++) sc[j] = 0.f;
            if (kb + (lane & 48) <= pos) {      // the 16 keys of a wave that skipped step 1 hold nothing
                for (int gg = 0; gg < H; gg++) {
                    const float x = rawl[lane * HP + gg];
#pragma unroll
                    for (int j = 0; j < HW; j++) {
                        const int h = wave + 4 * j;
                        if (h < H) sc[j] = fmaf(tk[h * H + gg], x, sc[j]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < HW; j++) {
                const int h = wave + 4 * j;
                if (h < H) {
                    const float v = see ? sc[j] : -INFINITY;
                    const float m_new = fmaxf(m_run[j], wave_max64(v));
                    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                    const float alpha = __expf(m_run[j] - m_safe);
                    const float e = __expf(v - m_safe);
                    l_run[j] = l_run[j] * alpha + wave_sum64(e);
                    m_run[j] = m_new;
                    ps2[((h / group) * 16 + h % group) * kDecPPitch + lane] = (bf16_t)e;
                    if (lane == 0) alv[h] = alpha;
                }
            }
        }
        __syncthreads();
        // ---- 3. outputs: this wave's value lanes, the heads of a key/value head as the columns
        {
            bf16x8_t vzero;
#pragma unroll
            for (int e = 0; e < 8; e++) vzero[e] = (bf16_t)0.f;
#pragma unroll
            for (int kvh = 0; kvh < kDecGMax; kvh++) {
                if (kvh < G) {
                    const int ha = kvh * group + c < H ? kvh * group + c : H - 1;
                    const float alpha = alv[ha];
#pragma unroll
                    for (int ts = 0; ts < TS; ts++) {
                        const int t = wave + 4 * ts;
                        if (t < DVT) {
                            f32x4_t acc = o[kvh][ts];
#pragma unroll
                            for (int i = 0; i < 4; i++) acc[i] *= alpha;
#pragma unroll
                            for (int s2 = 0; s2 < 2; s2++) {
                                if (kb + 32 * s2 > pos) continue;      // uniform: no key of this half is seen
                                const int key8 = kb + 32 * s2 + 8 * g;
                                bf16x8_t vf = vzero;
                                if (key8 <= pos) {
                                    const bf16x8_t v8 = *(const bf16x8_t *)(p.v_pages + (((size_t)vpage[s2] * G + kvh) * DV + 16 * t + c) * PS + key8 % PS);
#pragma unroll
                                    for (int e = 0; e < 8; e++) vf[e] = key8 + e <= pos ? v8[e] : (bf16_t)0.f;   // slots past the last token hold anything
                                }
                                const bf16x8_t pf = *(const bf16x8_t *)(ps2 + (kvh * 16 + c) * kDecPPitch + 32 * s2 + 8 * g);
                                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc, 0, 0, 0);
                            }
                            o[kvh][ts] = acc;
                        }
                    }
                }
            }
        }
        __syncthreads();   // rawl, ps2 and alv are rewritten by the next block
    }
#pragma unroll
    for (int j = 0; j < HW; j++) {
        const int h = wave + 4 * j;
        if (h < H && lane == 0) { mlv[h] = m_run[j]; mlv[H + h] = l_run[j]; }
    }
    __syncthreads();
    float *part = S > 1 ? p.ws + ((size_t)seg * S + split) * decode_part_floats(H, DV) : nullptr;
    if (S > 1 && tid < 2 * H) part[tid] = mlv[tid];
    if (c >= group) return;
#pragma unroll
    for (int kvh = 0; kvh < kDecGMax; kvh++) {
        if (kvh < G) {
            const int h = kvh * group + c;
#pragma unroll
            for (int ts = 0; ts < TS; ts++) {
                const int t = wave + 4 * ts;
                if (t >= DVT) continue;
                if (S > 1) {
                    *(f32x4_t *)(part + 2 * H + (size_t)h * DV + 16 * t + 4 * g) = o[kvh][ts];
                } else {
                    const float l = mlv[H + h];
                    float f = l > 0.f ? 1.0f / l : 0.f;
                    if (p.gate != nullptr) f *= 1.0f / (1.0f + __expf(-(float)p.gate[(size_t)r * p.gate_stride + h]));
                    bf16x4_t r4;
#pragma unroll
                    for (int i = 0; i < 4; i++) r4[i] = (bf16_t)(o[kvh][ts][i] * f);
                    *(bf16x4_t *)(p.out + (size_t)r * out_row + (size_t)h * DV + 16 * t + 4 * g) = r4;
                }
            }
        }
    }
}

// The shares of a decode row's workgroups into its output, a workgroup a (request, head): eight groups of 32 threads take
// every eighth share each (a thread four value lanes), then the eight partial merges meet in LDS.
__global__ void __launch_bounds__(kThreads) talking_decode_merge_kernel(const TalkArgs p) {
    __shared__ float gm[8], gl[8];
    __shared__ __attribute__((aligned(16))) float go[8][128];
    const int seg = blockIdx.x, h = blockIdx.y, H = p.heads, DV = p.v_dim, S = p.splits;
    const int r = seg;
    if (p.row_seg[r] < 0) return;      // a padding row: the decode kernel has written zeros
    const size_t per = decode_part_floats(H, DV);
    const float *parts = p.ws + (size_t)seg * S * per;
    const int sg = threadIdx.x >> 5, d4 = 4 * (threadIdx.x & 31);
    float m = -INFINITY, l = 0.f;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s = sg; s < S; s += 8) {
        const float *part = parts + s * per;
        const float ms = part[h], ls = part[H + h];
        f32x4_t o4 = {0.f, 0.f, 0.f, 0.f};
        if (d4 < DV) o4 = *(const f32x4_t *)(part + 2 * H + (size_t)h * DV + d4);
        if (ms == -INFINITY) continue;      // a share that saw no key
        const float m_new = fmaxf(m, ms);
        const float a = __expf(m - m_new), w = __expf(ms - m_new);      // m = -inf: a = 0
        l = l * a + ls * w;
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] = acc[e] * a + o4[e] * w;
        m = m_new;
    }
    if ((threadIdx.x & 31) == 0) { gm[sg] = m; gl[sg] = l; }
    if (d4 < DV) *(f32x4_t *)&go[sg][d4] = acc;
    __syncthreads();
    if (sg != 0 || d4 >= DV) return;
    float mt = -INFINITY;
#pragma unroll
    for (int k = 0; k < 8; k++) mt = fmaxf(mt, gm[k]);
    float lt = 0.f;
    f32x4_t tot = {0.f, 0.f, 0.f, 0.f};
    if (mt > -INFINITY) {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float w = __expf(gm[k] - mt);      // a group without a share: e^-inf = 0
            lt += gl[k] * w;
            const f32x4_t o4 = *(const f32x4_t *)&go[k][d4];
#pragma unroll
            for (int e = 0; e < 4; e++) tot[e] = fmaf(o4[e], w, tot[e]);
        }
    }
    float f = lt > 0.f ? 1.0f / lt : 0.f;
    if (p.gate != nullptr) f *= 1.0f / (1.0f + __expf(-(float)p.gate[(size_t)r * p.gate_stride + h]));
    bf16x4_t r4;
#pragma unroll
    for (int e = 0; e < 4; e++) r4[e] = (bf16_t)(tot[e] * f);
    *(bf16x4_t *)(p.out + (size_t)r * H * DV + (size_t)h * DV + d4) = r4;
}

// 1: not taken
int launch_decode(const TalkArgs &a, hipStream_t stream) {
    const int H = a.heads, G = a.kv_heads;
    if (H > 32 || G > kDecGMax || H / G > 16 || a.page_size % 8 != 0 || (H % 2 != 0 && a.splits > 1)) return 1;
    const int HP = H | 1;
    size_t floats = (size_t)H * H + (size_t)kKeyBlock * HP + 3 * H;
    floats = (floats + 3) & ~(size_t)3;
    const size_t lds = floats * sizeof(float) + ((size_t)H * a.k_dim + (size_t)G * 16 * kDecPPitch) * sizeof(bf16_t);
    if (lds > 60 * 1024) return 1;
    if (H <= 16) hipLaunchKernelGGL(talking_decode_kernel<4>, dim3(a.num_segs, a.splits), dim3(kThreads), lds, stream, a);
    else hipLaunchKernelGGL(talking_decode_kernel<8>, dim3(a.num_segs, a.splits), dim3(kThreads), lds, stream, a);
    int rc = fllm_check_launch("talking_attention (decode rows)");
    if (rc == 0 && a.splits > 1) {
        hipLaunchKernelGGL(talking_decode_merge_kernel, dim3(a.num_segs, H), dim3(kThreads), 0, stream, a);
        rc = fllm_check_launch("talking_attention (decode merge)");
    }
    return rc;
}

template <int HMAX>
int launch_tiles(const TalkArgs &a, int tiles, size_t lds, hipStream_t stream) {
    auto kernel = talking_tile_kernel<HMAX>;
    // the kernel's own arrays (mixing matrix, maxima, factors, weights) come on top of the queries and the stage: beyond
    // the default 64 KiB of both together the larger amount has to be asked for
    constexpr size_t own = sizeof(float) * (HMAX * HMAX + 5 * HMAX * kTileRows) + sizeof(bf16_t) * HMAX * 4 * kTileRows * 16 +
                           sizeof(int) * (kMaxSegsLds + 1);
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
        hipLaunchKernelGGL(talking_merge_kernel, dim3(tiles, a.heads), dim3(kThreads), 0, stream, a);
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
                                     int key_chunk, int max_context, int splits, float *ws, size_t ws_floats, int single_rows,
                                     hipStream_t stream) {
    if (key_chunk != 8 || k_dim % 32 != 0 || k_dim > 256 || v_dim % 16 != 0 || v_dim > 128 || heads > 16 || page_size % 4 != 0)
        return 1;
    // A stage holds as many key/value heads as a thread's 8 registers of 16 bytes and LDS allow, and the page numbers of
    // the keys a tile can see lie in LDS where they fit (up to 4,096: 65,536 keys of pages of 16).
    const int widest = k_dim > v_dim ? k_dim : v_dim;
    int gs = 256 / widest < kv_heads ? 256 / widest : kv_heads;
    const long span = chunk > 0 && chunk + 2 * kTileRows < max_context ? chunk + 2 * kTileRows : max_context;
    int ptab = (int)(span / page_size + 3);
    if (ptab > 4096) ptab = 0;
    auto lds_for = [&](int heads_a_stage, int pages) {
        const size_t k_elems = (size_t)kKeyBlock * (heads_a_stage * k_dim + 8), v_elems = (size_t)heads_a_stage * v_dim * kVPitch;
        const size_t stage = ((k_elems > v_elems ? k_elems : v_elems) + 7) & ~(size_t)7;
        return ((size_t)kTileRows * (heads * k_dim + 8) + stage) * sizeof(bf16_t) + (size_t)pages * sizeof(int);
    };
    constexpr size_t kLdsRoom = 160 * 1024 - 46 * 1024;      // what the kernel's own arrays leave at 16 heads
    while (gs > 1 && lds_for(gs, ptab) > kLdsRoom) gs--;
    if (lds_for(gs, ptab) > kLdsRoom) ptab = 0;
    const size_t lds = lds_for(gs, ptab);
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
    a.gs = gs;
    a.ptab = ptab;
    if (single_rows && rows == num_segs) {      // a decode step: every request has one row
        const int rc = launch_decode(a, stream);
        if (rc <= 0) return rc;
    }
    // every segment's rows in tiles of 16: at most rows / 16 full tiles and one ragged tile a segment
    const int tiles = rows / kTileRows + num_segs;
    // the kernel holds every head's scores and outputs of its rows in registers: an instance a head count bracket
    if (heads <= 8) return launch_tiles<8>(a, tiles, lds, stream);
    if (heads <= 12) return launch_tiles<12>(a, tiles, lds, stream);
    return launch_tiles<16>(a, tiles, lds, stream);
}
