// Many small products with one launch: out rows of group g = a rows . w[g]^T, where a group is a
// head (every row of the step, its own columns of `a` and of `out`) or an expert (the rows that a
// router sent to it, listed in tiles of kGroupedRows places by liyab_moe_align).
//
//   idx   = the row's number: m for heads; rows_list[place] for listed rows (-1: an empty place)
//   a row = a + (idx / a_div) * lda + g * a_group_cols       (a_div: entries a token, so that a
//                                                             token's row serves each of its experts)
//   w[g]  = w + g * N * K, a row an output feature ([N, K], K contiguous)
//   out   = out + (idx + (idx / out_div) * out_extra) * ldo + g * out_group_cols + column
//   value = acc0, or relu(acc0)^2 with act = 1   (one matrix)
//         = silu(acc0) * acc1                    (two matrices: a gated unit's first products)
//     then * row_scale[idx] (a router's weight), * sigmoid(gate[idx * gate_stride + g * N + column])
//     (the gate's logits float32 or bfloat16)
//
// bfloat16 operands with K a multiple of 8 run on the matrix cores in tiles of 64 x 64 (four waves
// of 32 x 32, K in steps of 64 through LDS, 32-bit sums); float32 operands, and sizes the matrix
// kernel does not take, run as plain multiply-adds in 32-bit (tiles of 64 x 64, a thread 4 x 4).
// Every output element is a sum over k in one order whatever rows share its tile.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kGroupedRows = 64;  // rows a tile; liyab_moe_align lays its lists out in these,
constexpr int kSkinnyRows = 16;   // or in these for steps whose experts get few rows each

struct GroupedParams {
    const void* a;
    int64_t lda;
    int a_div, a_group_cols;
    const void* w0;
    const void* w1;
    void* out;
    int64_t ldo;
    int out_group_cols, out_dtype;
    const int* rows_list;   // null: rows 0..M-1 and the group is blockIdx.z
    const int* tile_group;  // with rows_list: the group of each tile of rows, -1 for a tile nobody uses
    const float* row_scale;
    const void* gate;  // logits of a gate on the output, float32 or bfloat16 (gate_dtype), or null
    int64_t gate_stride;
    int gate_dtype;
    int M, N, K;
    int block;  // places a tile of rows_list: kGroupedRows, or kSkinnyRows for steps of few rows
    int act;        // one matrix: 0 = the sums as they are, 1 = the square of their positive part (relu(.)^2)
    int out_div, out_extra;  // `out_extra` rows of `out` are left free behind each `out_div` rows (a token's entries), for results another product adds
};

__device__ __forceinline__ float gp_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <int NW>
__device__ __forceinline__ void grouped_store(const GroupedParams& p, int idx, int g, int n, float v0, float v1) {
    float v = v0;
    if constexpr (NW == 2) v = v0 * gp_sigmoid(v0) * v1;
    else if (p.act == 1) v = v0 > 0.0f ? v0 * v0 : 0.0f;
    if (p.row_scale != nullptr) v *= p.row_scale[idx];
    if (p.gate != nullptr) {
        const int64_t ga = static_cast<int64_t>(idx) * p.gate_stride + static_cast<int64_t>(g) * p.N + n;
        v *= gp_sigmoid(p.gate_dtype == kF32 ? static_cast<const float*>(p.gate)[ga] : bf16_to_float(static_cast<const bf16_t*>(p.gate)[ga]));
    }
    const int64_t at = static_cast<int64_t>(idx + (idx / p.out_div) * p.out_extra) * p.ldo + static_cast<int64_t>(g) * p.out_group_cols + n;
    if (p.out_dtype == kF32)
        static_cast<float*>(p.out)[at] = v;
    else
        static_cast<bf16_t*>(p.out)[at] = float_to_bf16(v);
}

// The rows of this workgroup's tile: their numbers into `idx` (LDS, kGroupedRows ints), the group returned (-1: nothing to do).
__device__ __forceinline__ int grouped_rows(const GroupedParams& p, int* idx) {
    const int tile = blockIdx.x;
    int g;
    if (p.rows_list != nullptr) {
        g = p.tile_group[tile];
        if (g < 0) return -1;
        for (int i = threadIdx.x; i < kGroupedRows; i += blockDim.x) idx[i] = i < p.block ? p.rows_list[tile * p.block + i] : -1;
    } else {
        g = blockIdx.z;
        for (int i = threadIdx.x; i < kGroupedRows; i += blockDim.x) {
            const int m = tile * kGroupedRows + i;
            idx[i] = m < p.M ? m : -1;
        }
    }
    __syncthreads();
    return g;
}

typedef __attribute__((ext_vector_type(8))) __bf16 gp_bf16x8;
typedef __attribute__((ext_vector_type(16))) float gp_floatx16;
typedef __attribute__((ext_vector_type(4))) uint32_t gp_u32x4;

constexpr int GPK = 64;       // k per LDS tile
constexpr int GPLD = GPK + 8;  // padded row, in elements

template <int NW>
__global__ void __launch_bounds__(256)
grouped_mfma_kernel(GroupedParams p) {
    __shared__ __attribute__((aligned(16))) bf16_t lds[(1 + NW) * 64 * GPLD];
    __shared__ int idx[kGroupedRows];
    const int g = grouped_rows(p, idx);
    if (g < 0) return;
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave / 2, wn = wave % 2;
    const int n0 = blockIdx.y * 64;
    const int li = lane % 32, lk = (lane / 32) * 8;
    const int N = p.N, K = p.K;
    const bf16_t* a = static_cast<const bf16_t*>(p.a) + static_cast<int64_t>(g) * p.a_group_cols;
    const bf16_t* w[2] = {static_cast<const bf16_t*>(p.w0) + static_cast<int64_t>(g) * N * K,
                          NW == 2 ? static_cast<const bf16_t*>(p.w1) + static_cast<int64_t>(g) * N * K : nullptr};
    gp_floatx16 acc[NW];
#pragma unroll
    for (int u = 0; u < NW; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[u][r] = 0.0f;

    // a thread's two 16-byte pieces of each operand tile: rows tid / 8 and tid / 8 + 32, k piece tid % 8.
    // Every load is made, from a row that exists (an empty place reads the first row, a feature past N the
    // first feature, a piece past K the row's last piece) and masked afterwards: a load under a branch is
    // waited for where the branch ends, and the pieces of kStages tiles of K are to be in flight together.
    const int row_a = tid / 8, kc = (tid % 8) * 8;
    const bf16_t* a_src[2];
    const bf16_t* w_src[NW][2];
    bool a_ok[2], w_ok[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int id = idx[row_a + 32 * i];
        a_ok[i] = id >= 0;
        a_src[i] = a + static_cast<int64_t>(a_ok[i] ? id / p.a_div : 0) * p.lda;
        const int n = n0 + row_a + 32 * i;
        w_ok[i] = n < N;
#pragma unroll
        for (int u = 0; u < NW; ++u) w_src[u][i] = w[u] + static_cast<int64_t>(w_ok[i] ? n : 0) * K;
    }
    const gp_u32x4 zero = {0, 0, 0, 0};
    constexpr int kStages = NW == 2 ? 1 : 2;  // tiles of K whose pieces are in flight: a tile's trip from memory is most of its time otherwise
    gp_u32x4 ra[kStages][2], rw[kStages][NW][2];
    auto fetch = [&](int s, int k0) {
        const int k = min(k0 + kc, K - 8);
        const bool in_k = k0 + kc < K;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const gp_u32x4 va = *reinterpret_cast<const gp_u32x4*>(a_src[i] + k);
            ra[s][i] = (a_ok[i] && in_k) ? va : zero;
#pragma unroll
            for (int u = 0; u < NW; ++u) {
                const gp_u32x4 vw = *reinterpret_cast<const gp_u32x4*>(w_src[u][i] + k);
                rw[s][u][i] = (w_ok[i] && in_k) ? vw : zero;
            }
        }
    };
    const int nk = (K + GPK - 1) / GPK;
#pragma unroll
    for (int s = 0; s < kStages; ++s) fetch(s, min(s, nk - 1) * GPK);  // (a stage past the last tile reads the last one again, unused)
    for (int kb = 0; kb < nk; kb += kStages) {
#pragma unroll
        for (int s = 0; s < kStages; ++s) {
            if (kb + s < nk) {  // (the same for every thread of the workgroup)
                lds_barrier();  // the previous tile's fragments have been read
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    *reinterpret_cast<gp_u32x4*>(lds + (row_a + 32 * i) * GPLD + kc) = ra[s][i];
#pragma unroll
                    for (int u = 0; u < NW; ++u) *reinterpret_cast<gp_u32x4*>(lds + ((1 + u) * 64 + row_a + 32 * i) * GPLD + kc) = rw[s][u][i];
                }
                fetch(s, min(kb + s + kStages, nk - 1) * GPK);
                lds_barrier();
                const bf16_t* Ab = lds + (wm * 32 + li) * GPLD + lk;
#pragma unroll
                for (int ks = 0; ks < GPK; ks += 16) {
                    const gp_bf16x8 fa = *reinterpret_cast<const gp_bf16x8*>(Ab + ks);
#pragma unroll
                    for (int u = 0; u < NW; ++u) {
                        const gp_bf16x8 fw = *reinterpret_cast<const gp_bf16x8*>(lds + ((1 + u) * 64 + wn * 32 + li) * GPLD + lk + ks);
                        acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fw, acc[u], 0, 0, 0);
                    }
                }
            }
        }
    }
    // C block layout: a lane holds column li; rows 8 * (r / 4) + 4 * (lane / 32) + r % 4
    const int n = n0 + wn * 32 + li;
    if (n >= N) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int id = idx[wm * 32 + 4 * (lane / 32) + 8 * (r / 4) + r % 4];
        if (id >= 0) grouped_store<NW>(p, id, g, n, acc[0][r], NW == 2 ? acc[NW - 1][r] : 0.0f);
    }
}

// Few rows a group (decoding: an expert gets a token or two): the product is a stream of the group's
// weights, and what matters is how many workgroups pull on it. A workgroup owns 16 output features and one
// tile of 16 row places; its four waves deal the units of 64 k among themselves and add their sums through
// LDS in wave order. With v_mfma_f32_16x16x32_bf16 the weights are the first operand and the rows the second,
// both straight from global memory into registers, 16 bytes a lane, a trip ahead of the multiplies. The order
// of an element's sum depends on K alone.
typedef __attribute__((ext_vector_type(4))) float gp_floatx4;
union GpFrag {
    gp_u32x4 u;
    gp_bf16x8 v;
};

template <int NW>
__global__ void __launch_bounds__(256)
grouped_skinny_kernel(GroupedParams p) {
    __shared__ float red[4 * NW * 256];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, q = lane / 16;
    const int tile = blockIdx.x;
    int g;
    if (p.rows_list != nullptr) {
        g = p.tile_group[tile];
        if (g < 0) return;
    } else {
        g = blockIdx.z;
    }
    auto row_id = [&](int place) {
        if (p.rows_list != nullptr) return p.rows_list[tile * kSkinnyRows + place];
        const int m = tile * kSkinnyRows + place;
        return m < p.M ? m : -1;
    };
    const int N = p.N, K = p.K, n0 = blockIdx.y * 16;
    const int my_id = row_id(i);
    // an empty place reads the first row, a feature past N the last one: computed, never stored
    const bf16_t* arow = static_cast<const bf16_t*>(p.a) + static_cast<int64_t>(my_id >= 0 ? my_id / p.a_div : 0) * p.lda + static_cast<int64_t>(g) * p.a_group_cols;
    const int64_t wrow = (static_cast<int64_t>(g) * N + min(n0 + i, N - 1)) * K;
    const bf16_t* w[2] = {static_cast<const bf16_t*>(p.w0) + wrow, NW == 2 ? static_cast<const bf16_t*>(p.w1) + wrow : nullptr};
    const gp_u32x4 zero = {0, 0, 0, 0};
    // a lane's two pieces of a unit of 64 k: k0 + 8 q and k0 + 32 + 8 q; a piece past K reads the row's last piece, as zeros for the weights
    auto fetch = [&](int unit, GpFrag (&x)[2], GpFrag (&wf)[NW][2]) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = unit * 64 + 32 * h + 8 * q;
            const int kk = min(k, K - 8);
            x[h].u = *reinterpret_cast<const gp_u32x4*>(arow + kk);
#pragma unroll
            for (int u = 0; u < NW; ++u) {
                const gp_u32x4 v = *reinterpret_cast<const gp_u32x4*>(w[u] + kk);
                wf[u][h].u = k < K ? v : zero;
            }
        }
    };
    gp_floatx4 acc[NW];
#pragma unroll
    for (int u = 0; u < NW; ++u) acc[u] = gp_floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    const int units = (K + 63) / 64;
    GpFrag xc[2], wc[NW][2];
    int unit = wave;
    if (unit < units) fetch(unit, xc, wc);
    while (unit < units) {  // (the same trips for every lane of a wave)
        const int next = unit + 4;
        GpFrag xn[2], wn[NW][2];
        if (next < units) fetch(next, xn, wn);
#pragma unroll
        for (int u = 0; u < NW; ++u) {
            acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[u][0].v, xc[0].v, acc[u], 0, 0, 0);
            acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[u][1].v, xc[1].v, acc[u], 0, 0, 0);
        }
        if (next < units) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                xc[h] = xn[h];
#pragma unroll
                for (int u = 0; u < NW; ++u) wc[u][h] = wn[u][h];
            }
        }
        unit = next;
    }
    // acc[u][r] = this wave's share of C^T[n = 4 q + r][m = i]; kept [wave][matrix][m][n]
#pragma unroll
    for (int u = 0; u < NW; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[(wave * NW + u) * 256 + i * 16 + 4 * q + r] = acc[u][r];
    __syncthreads();
    const int m = tid / 16, n = n0 + tid % 16;
    float v[2] = {0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < NW; ++u)
#pragma unroll
        for (int wv = 0; wv < 4; ++wv) v[u] += red[(wv * NW + u) * 256 + tid];
    const int id = row_id(m);
    if (id >= 0 && n < N) grouped_store<NW>(p, id, g, n, v[0], v[1]);
}

// Plain 32-bit multiply-adds: a tile of 64 rows x 64 output features, a thread 4 x 4 of them, K in
// steps of 16 through LDS. Takes every size and both element types.
template <typename T, int NW>
__global__ void __launch_bounds__(256)
grouped_plain_kernel(GroupedParams p) {
    constexpr int BK = 16;
    __shared__ float la[BK][64 + 1];
    __shared__ float lw[NW][BK][64 + 1];
    __shared__ int idx[kGroupedRows];
    const int g = grouped_rows(p, idx);
    if (g < 0) return;
    const int tid = threadIdx.x;
    const int n0 = blockIdx.y * 64;
    const int N = p.N, K = p.K;
    const T* a = static_cast<const T*>(p.a) + static_cast<int64_t>(g) * p.a_group_cols;
    const T* w[2] = {static_cast<const T*>(p.w0) + static_cast<int64_t>(g) * N * K,
                     NW == 2 ? static_cast<const T*>(p.w1) + static_cast<int64_t>(g) * N * K : nullptr};
    const int tr = (tid / 16) * 4, tc = (tid % 16) * 4;  // this thread's rows and columns of the tile
    float acc[NW][4][4];
#pragma unroll
    for (int u = 0; u < NW; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[u][i][j] = 0.0f;
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();
        // 64 x 16 values of each operand: a thread four of them, k fastest
        for (int e = tid; e < 64 * BK; e += 256) {
            const int row = e / BK, k = k0 + e % BK;
            const int id = idx[row];
            la[e % BK][row] = (id >= 0 && k < K) ? to_float<T>(a[static_cast<int64_t>(id / p.a_div) * p.lda + k]) : 0.0f;
            const int n = n0 + row;
#pragma unroll
            for (int u = 0; u < NW; ++u) lw[u][e % BK][row] = (n < N && k < K) ? to_float<T>(w[u][static_cast<int64_t>(n) * K + k]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float av[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = la[k][tr + i];
#pragma unroll
            for (int u = 0; u < NW; ++u) {
                float wv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) wv[j] = lw[u][k][tc + j];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[u][i][j] = fmaf(av[i], wv[j], acc[u][i][j]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int id = idx[tr + i];
        if (id < 0) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tc + j;
            if (n < N) grouped_store<NW>(p, id, g, n, acc[0][i][j], NW == 2 ? acc[NW - 1][i][j] : 0.0f);
        }
    }
}

}  // namespace liyab

using namespace liyab;

// See the head of this file. dtype: the element type of a, w0 and w1. n_groups: heads (rows_list
// null) or experts (the values of tile_group lie below it; the caller has made them so). n_tiles:
// the tiles of rows to launch (with rows_list: the length of tile_group; without: (M + block - 1) / block).
// block: the row places a tile, 64, or 16 for steps of few rows a group (bfloat16 operands in 16-byte pieces).
extern "C" int liyab_grouped_product(const void* a, int64_t lda, int a_div, int a_group_cols, const void* w0, const void* w1, int dtype,
                                     void* out, int out_dtype, int64_t ldo, int out_group_cols, const int* rows_list,
                                     const int* tile_group, int n_tiles, int block, int n_groups, const float* row_scale,
                                     const void* gate, int gate_dtype, int64_t gate_stride, int M, int N, int K, int act, int out_div, int out_extra,
                                     hipStream_t stream) {
    LIYAB_REQUIRE(a && w0 && out, "grouped_product: null pointer");
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "grouped_product: unknown dtype %d", dtype);
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "grouped_product: unknown output dtype %d", out_dtype);
    LIYAB_REQUIRE(M >= 0 && N > 0 && K > 0 && a_div >= 1 && n_groups >= 1 && n_groups <= 65535 && n_tiles >= 0, "grouped_product: bad sizes M=%d N=%d K=%d", M, N, K);
    LIYAB_REQUIRE((rows_list == nullptr) == (tile_group == nullptr), "grouped_product: a list of rows goes with the groups of its tiles");
    LIYAB_REQUIRE(block == kGroupedRows || block == kSkinnyRows, "grouped_product: tiles of %d rows (%d or %d)", block, kGroupedRows, kSkinnyRows);
    LIYAB_REQUIRE(rows_list != nullptr || n_tiles == (M + block - 1) / block, "grouped_product: %d tiles for %d rows", n_tiles, M);
    LIYAB_REQUIRE(gate == nullptr || gate_dtype == kF32 || gate_dtype == kBF16, "grouped_product: unknown gate dtype %d", gate_dtype);
    LIYAB_REQUIRE(gate == nullptr || gate_stride >= static_cast<int64_t>(rows_list ? 1 : n_groups) * N, "grouped_product: the gate's rows are shorter than the output's");
    LIYAB_REQUIRE((act == 0 || (act == 1 && w1 == nullptr)) && out_div >= 1 && out_extra >= 0, "grouped_product: unknown activation %d, or one beside a gated unit", act);
    if (M == 0 || n_tiles == 0) return 0;
    GroupedParams p{a, lda, a_div, a_group_cols, w0, w1, out, ldo, out_group_cols, out_dtype, rows_list, tile_group, row_scale, gate, gate_stride, gate_dtype, M, N, K, block, act, out_div, out_extra};
    const dim3 grid(n_tiles, (N + 63) / 64, rows_list ? 1 : n_groups);
    const bool matrix = dtype == kBF16 && K % 8 == 0 && lda % 8 == 0 && a_group_cols % 8 == 0 &&
                        (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w0) & 15) == 0 &&
                        (reinterpret_cast<uintptr_t>(w1) & 15) == 0;
    LIYAB_REQUIRE(block == kGroupedRows || matrix, "grouped_product: tiles of %d rows are for bfloat16 operands in 16-byte pieces", kSkinnyRows);
    if (block == kSkinnyRows) {
        const dim3 skinny(n_tiles, (N + 15) / 16, rows_list ? 1 : n_groups);
        if (w1 != nullptr) grouped_skinny_kernel<2><<<skinny, 256, 0, stream>>>(p);
        else grouped_skinny_kernel<1><<<skinny, 256, 0, stream>>>(p);
    } else if (matrix) {
        if (w1 != nullptr) grouped_mfma_kernel<2><<<grid, 256, 0, stream>>>(p);
        else grouped_mfma_kernel<1><<<grid, 256, 0, stream>>>(p);
    } else if (dtype == kBF16) {
        if (w1 != nullptr) grouped_plain_kernel<bf16_t, 2><<<grid, 256, 0, stream>>>(p);
        else grouped_plain_kernel<bf16_t, 1><<<grid, 256, 0, stream>>>(p);
    } else {
        if (w1 != nullptr) grouped_plain_kernel<float, 2><<<grid, 256, 0, stream>>>(p);
        else grouped_plain_kernel<float, 1><<<grid, 256, 0, stream>>>(p);
    }
    return check_launch("grouped_product");
}
