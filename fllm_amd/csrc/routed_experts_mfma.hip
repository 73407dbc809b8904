// Routed experts on the matrix cores (bfloat16, prompt portions): the (row, pick) pairs of a step are grouped by expert on
// the device, and every expert multiplies the rows that picked it as tiles of 64 rows, so that its matrices are read once
// a row tile instead of once a row.  Three launches: grouping, gate/up with the activation, down.  A pair's result does not
// depend on which rows share its tile (a row of a matrix-core product is a sum over K in an order of its own).
//
// MFMA operand layout used here (wave64, v_mfma_f32_32x32x16_bf16): A lane l holds A[m = l%32][k = 8*(l/32) .. +7]; B
// likewise with n = l%32; D lane l holds D[m = 8*(i/4) + 4*(l/32) + i%4][n = l%32], i = 0..15.
#include "api.h"
#include "common.h"

namespace {

constexpr int GM = 64;              // pairs a row tile
constexpr int GN = 128;             // weight rows a column tile: 128 outputs, or 64 gate rows and the same 64 up rows
constexpr int GK = 64, LDT = GK + 8;
constexpr int kThreads = 256;

__device__ __forceinline__ bf16x8_t zero8() {
    bf16x8_t z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.0f;
    return z;
}

// One workgroup.  counts -> first pair slot and first tile of every expert -> the pairs of an expert side by side in
// `order`, and a list of tiles (expert, first slot, pairs).  work: [0] number of tiles, then 3 ints a tile, then order.
__global__ void __launch_bounds__(1024)
group_pairs_kernel(const int32_t *__restrict__ ids, int pairs, int E, int max_tiles, int32_t *__restrict__ work) {
    extern __shared__ int lds[];      // count[E], slot[E], tile[E]
    int *count = lds, *slot = lds + E, *tile = lds + 2 * E;
    int32_t *tiles = work + 1, *order = work + 1 + 3 * max_tiles;
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        int e = ids[p];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int s = 0, t = 0;
        for (int e = 0; e < E; e++) {
            slot[e] = s;
            tile[e] = t;
            s += count[e];
            t += (count[e] + GM - 1) / GM;
        }
        work[0] = t;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int n = count[e];
        for (int i = 0, t = tile[e]; i < n; i += GM, t++) {
            tiles[3 * t] = e;
            tiles[3 * t + 1] = slot[e] + i;
            tiles[3 * t + 2] = n - i < GM ? n - i : GM;
        }
    }
    __syncthreads();       // slot[] becomes the cursor of its expert
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        int e = ids[p];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        order[atomicAdd(&slot[e], 1)] = p;
    }
}

// MODE 0: act[pair, c] = a(g) * (u + up_offset) for 64 columns c a workgroup; A rows = h[pair / top] * weights[pair],
//         rounded to bfloat16; B = 64 gate rows and 64 up rows of the expert.  w: [E][2 N][K].
// MODE 1: out[pair, c] = w[e][c] . act[pair] for 128 columns, float32.  w: [E][N][K].
template <int MODE>
__global__ void __launch_bounds__(kThreads)
grouped_tiles_kernel(const bf16_t *__restrict__ x, int ldx, const float *__restrict__ weights, int top, const int32_t *__restrict__ work,
                     int max_tiles, const bf16_t *__restrict__ w, int N, int K, bf16_t *__restrict__ act, float *__restrict__ out,
                     float limit, float alpha, float up_offset) {
    __shared__ __attribute__((aligned(16))) bf16_t As[GM * LDT];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[GN * LDT];
    __shared__ int s_pair[GM];
    __shared__ float s_scale[GM];
    const int t = blockIdx.x % max_tiles, tn = blockIdx.x / max_tiles;     // neighbouring workgroups share a column tile
    if (t >= work[0]) return;
    const int32_t *tile = work + 1 + 3 * t, *order = work + 1 + 3 * max_tiles;
    const int e = tile[0], first = tile[1], count = tile[2];
    constexpr int COLS = MODE == 0 ? GN / 2 : GN;      // output columns a workgroup
    const int n0 = tn * COLS;
    if (threadIdx.x < GM) {
        const int pair = threadIdx.x < count ? order[first + threadIdx.x] : -1;
        s_pair[threadIdx.x] = pair;
        s_scale[threadIdx.x] = (MODE == 0 && pair >= 0) ? weights[pair] : 1.0f;
    }
    __syncthreads();
    const bf16_t *wb = w + (size_t)e * (MODE == 0 ? 2 : 1) * N * K;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lg = lane >> 5;

    f32x16_t acc[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[j][v] = 0.f;

    constexpr int kA = (GM * GK / 8) / kThreads, kB = (GN * GK / 8) / kThreads;     // 16-byte chunks a thread: 2 and 4
    bf16x8_t ra[kA], rb[kB];
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int c = 0; c < kA; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            const int row = chunk / (GK / 8), k = k0 + (chunk % (GK / 8)) * 8;
            const int pair = s_pair[row];
            bf16x8_t v = zero8();
            if (pair >= 0 && k < K) {
                v = *(const bf16x8_t *)(x + (size_t)(MODE == 0 ? pair / top : pair) * ldx + k);
                if (MODE == 0) {
                    const float s = s_scale[row];
#pragma unroll
                    for (int i = 0; i < 8; i++) v[i] = (bf16_t)((float)v[i] * s);
                }
            }
            ra[c] = v;
        }
#pragma unroll
        for (int c = 0; c < kB; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            const int row = chunk / (GK / 8), k = k0 + (chunk % (GK / 8)) * 8;
            // MODE 0: rows 0..63 are gate rows n0 .., rows 64..127 the up rows of the same columns
            const int col = MODE == 0 ? n0 + (row & (COLS - 1)) : n0 + row;
            const size_t wrow = MODE == 0 ? (size_t)(row >= COLS ? N : 0) + col : (size_t)col;
            rb[c] = (col < N && k < K) ? *(const bf16x8_t *)(wb + wrow * K + k) : zero8();
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int c = 0; c < kA; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            *(bf16x8_t *)(As + (chunk / (GK / 8)) * LDT + (chunk % (GK / 8)) * 8) = ra[c];
        }
#pragma unroll
        for (int c = 0; c < kB; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            *(bf16x8_t *)(Bs + (chunk / (GK / 8)) * LDT + (chunk % (GK / 8)) * 8) = rb[c];
        }
    };
    // the wave's two product columns: MODE 0 the gate and the up rows of its 32 columns, MODE 1 two runs of 32 columns
    const int brow0 = MODE == 0 ? wn * 32 + l32 : wn * 64 + l32;
    const int brow1 = MODE == 0 ? COLS + wn * 32 + l32 : wn * 64 + 32 + l32;

    load_tile(0);
    for (int k0 = 0; k0 < K; k0 += GK) {
        store_tile();
        __syncthreads();
        if (k0 + GK < K) load_tile(k0 + GK);   // in flight while this tile is multiplied
#pragma unroll
        for (int kk = 0; kk < GK / 16; kk++) {
            const bf16x8_t a = *(const bf16x8_t *)(As + (wm * 32 + l32) * LDT + kk * 16 + lg * 8);
            const bf16x8_t b0 = *(const bf16x8_t *)(Bs + brow0 * LDT + kk * 16 + lg * 8);
            const bf16x8_t b1 = *(const bf16x8_t *)(Bs + brow1 * LDT + kk * 16 + lg * 8);
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[1], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int pair = s_pair[wm * 32 + 8 * (v / 4) + 4 * lg + (v % 4)];
        if (pair < 0) continue;
        if (MODE == 0) {
            const int n = n0 + wn * 32 + l32;
            if (n >= N) continue;
            float g = acc[0][v], u = acc[1][v];
            if (limit > 0.f) {
                g = fminf(g, limit);
                u = fminf(fmaxf(u, -limit), limit);
            }
            act[(size_t)pair * N + n] = (bf16_t)(g / (1.0f + expf(-alpha * g)) * (u + up_offset));
        } else {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int n = n0 + wn * 64 + j * 32 + l32;
                if (n < N) out[(size_t)pair * N + n] = acc[j][v];
            }
        }
    }
}

}  // namespace

// ints of scratch that fllm_experts_grouped needs for `pairs` (row, pick) pairs over E experts
extern "C" size_t fllm_experts_grouped_work_ints(int pairs, int E) {
    const size_t max_tiles = (size_t)(pairs + GM - 1) / GM + E;
    return 1 + 3 * max_tiles + pairs;
}

// 0: launched, negative: error, 1: shape declined (the caller runs the plain kernels).  h bfloat16 [rows, K] (row stride ldh);
// ids / weights [rows, top]; w_gate_up [E][2 inter][K]; w_down [E][N][inter]; act bfloat16 [rows * top, inter] (scratch);
// out float32 [rows * top, N]; work: fllm_experts_grouped_work_ints() int32.
extern "C" int fllm_experts_grouped(const void *h, int ldh, const int32_t *ids, const float *weights, int rows, int top,
                                    const void *w_gate_up, const void *w_down, int E, int inter, int K, int N, void *act, float *out,
                                    int32_t *work, float limit, float alpha, float up_offset, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && top > 0 && E > 0 && inter > 0 && K > 0 && N > 0 && ldh >= K, "experts_grouped: bad sizes");
    FLLM_REQUIRE(h && ids && weights && w_gate_up && w_down && act && out && work, "experts_grouped: operands missing");
    if (!fllm_fast_kernels_enabled()) return 1;
    if (K % 8 != 0 || inter % 8 != 0 || ldh % 8 != 0 || E > 4096) return 1;
    if ((((uintptr_t)h | (uintptr_t)w_gate_up | (uintptr_t)w_down | (uintptr_t)act) & 15) != 0) return 1;
    const long pairs = (long)rows * top;
    if (pairs == 0) return 0;
    const long max_tiles = (pairs + GM - 1) / GM + E;
    const long up_tiles = (inter + GN / 2 - 1) / (GN / 2), down_tiles = (N + GN - 1) / GN;
    if (pairs > (1L << 24) || max_tiles * up_tiles > 0x7fffffffL || max_tiles * down_tiles > 0x7fffffffL) return 1;
    hipLaunchKernelGGL(group_pairs_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), stream, ids, (int)pairs, E, (int)max_tiles, work);
    hipLaunchKernelGGL(grouped_tiles_kernel<0>, dim3((unsigned)(max_tiles * up_tiles)), dim3(kThreads), 0, stream, (const bf16_t *)h, ldh,
                       weights, top, work, (int)max_tiles, (const bf16_t *)w_gate_up, inter, K, (bf16_t *)act, nullptr, limit, alpha,
                       up_offset);
    hipLaunchKernelGGL(grouped_tiles_kernel<1>, dim3((unsigned)(max_tiles * down_tiles)), dim3(kThreads), 0, stream, (const bf16_t *)act,
                       inter, nullptr, 1, work, (int)max_tiles, (const bf16_t *)w_down, N, inter, nullptr, out, 0.f, 0.f, 0.f);
    return fllm_check_launch("experts_grouped");
}
