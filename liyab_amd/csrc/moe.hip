// Routing of a mixture of experts: who goes where, before the experts' products run
// (grouped_product.hip).
//
// liyab_moe_route: from each token's 32-bit router logits the `top` experts with the largest
// logits (among equal logits the lower number first) and their weights, the softmax over the chosen
// logits alone, in 32-bit. ids and weights [n, top]: entry t * top + k is token t's k-th choice.
// mode 1: the choice among groups of experts instead (route_token_groups): softmax over all experts, the best
// groups only, weights divided by their sum.
//
// liyab_moe_align: the entries listed by expert, each expert's stretch padded to whole tiles of
// `block` places: rows_list [max_tiles * block] (an entry's number, -1 for an empty place) and
// tile_group [max_tiles] (the expert of each tile, -1 for a tile that is not used). max_tiles is
// a bound that the step's sizes fix (entries / block + min(experts, entries), rounded up), so
// that the products' grids do not depend on where the tokens went. One workgroup.
//
// liyab_moe_route_align: both in one launch, for steps of at most 1,024 tokens.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kMaxTop = 64;

// One token's choice: the `top` largest of its E logits (the lower number among equals) and the softmax over them.
__device__ __forceinline__ void route_token(const float* __restrict__ z, int E, int top, int* __restrict__ ids, float* __restrict__ weights) {
    int chosen[kMaxTop];
    float value[kMaxTop];
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = 0.0f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken = taken || chosen[j] == e;
            const float v = z[e];
            if (!taken && (best < 0 || v > bv)) {
                best = e;
                bv = v;
            }
        }
        chosen[k] = best;
        value[k] = bv;
    }
    float sum = 0.0f;
    const float largest = value[0];  // the first choice holds the largest logit
    for (int k = 0; k < top; ++k) {
        value[k] = expf(value[k] - largest);
        sum += value[k];
    }
    for (int k = 0; k < top; ++k) {
        ids[k] = chosen[k];
        weights[k] = value[k] / sum;
    }
}

// One token's choice among groups of experts: s = softmax(z) over all experts; the experts form `n_groups` equal groups of
// neighbours, a group's score is its largest s, and only experts of the `keep` best groups (the lower number among equals)
// can be chosen; of those the `top` largest s (the lower number among equals), weighted s / (their sum + 1e-20).
constexpr int kMaxGroups = 64;
constexpr float kWeightFloor = 1e-20f;

__device__ __forceinline__ void route_token_groups(const float* __restrict__ z, int E, int top, int n_groups, int keep, int* __restrict__ ids,
                                                   float* __restrict__ weights) {
    float largest = z[0];
    for (int e = 1; e < E; ++e) largest = fmaxf(largest, z[e]);
    float total = 0.0f;
    for (int e = 0; e < E; ++e) total += expf(z[e] - largest);
    const int per = E / n_groups;
    uint64_t kept = 0;  // the groups whose experts can be chosen
    for (int k = 0; k < keep; ++k) {
        int best = -1;
        float bv = 0.0f;
        for (int g = 0; g < n_groups; ++g) {
            if ((kept >> g) & 1) continue;
            float gv = z[g * per];
            for (int e = 1; e < per; ++e) gv = fmaxf(gv, z[g * per + e]);  // (the largest score is the largest logit's)
            if (best < 0 || gv > bv) {
                best = g;
                bv = gv;
            }
        }
        kept |= uint64_t(1) << best;
    }
    int chosen[kMaxTop];
    float value[kMaxTop];
    float sum = 0.0f;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = 0.0f;
        for (int e = 0; e < E; ++e) {
            if (!((kept >> (e / per)) & 1)) continue;
            bool taken = false;
            for (int j = 0; j < k; ++j) taken = taken || chosen[j] == e;
            const float v = z[e];
            if (!taken && (best < 0 || v > bv)) {
                best = e;
                bv = v;
            }
        }
        chosen[k] = best;
        value[k] = expf(bv - largest) / total;
        sum += value[k];
    }
    for (int k = 0; k < top; ++k) {
        ids[k] = chosen[k];
        weights[k] = value[k] / (sum + kWeightFloor);
    }
}

// mode 0: the largest logits, softmax over the chosen ones; mode 1: softmax over all, groups, weights by their sum
__device__ __forceinline__ void route_any(const float* __restrict__ z, int E, int top, int mode, int n_groups, int keep, int* __restrict__ ids,
                                          float* __restrict__ weights) {
    if (mode == 1) route_token_groups(z, E, top, n_groups, keep, ids, weights);
    else route_token(z, E, top, ids, weights);
}

__global__ void __launch_bounds__(256)
moe_route_kernel(const float* __restrict__ logits, int64_t ld, int n, int E, int top, int* __restrict__ ids, float* __restrict__ weights,
                 int mode, int n_groups, int keep) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= n) return;
    route_any(logits + static_cast<int64_t>(t) * ld, E, top, mode, n_groups, keep, ids + static_cast<int64_t>(t) * top, weights + static_cast<int64_t>(t) * top);
}

// The entries of `ids` listed by expert in tiles of `block` places; one workgroup of 1,024 threads runs this.
__device__ __forceinline__ void align_entries(const int* __restrict__ ids, int n_entries, int E, int block, int* __restrict__ rows_list,
                                              int* __restrict__ tile_group, int max_tiles, int* sh) {
    int* counts = sh;     // [E]
    int* first = sh + E;  // [E + 1]: the first place of each expert
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 1024) counts[e] = 0;
    for (int i = tid; i < max_tiles * block; i += 1024) rows_list[i] = -1;
    for (int i = tid; i < max_tiles; i += 1024) tile_group[i] = -1;
    __syncthreads();
    for (int i = tid; i < n_entries; i += 1024) {
        const int e = ids[i];
        if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at;
            const int tiles = (counts[e] + block - 1) / block;
            for (int i = 0; i < tiles; ++i)
                if (at / block + i < max_tiles) tile_group[at / block + i] = e;
            at += tiles * block;
            counts[e] = 0;  // counts the entries placed so far from here on
        }
        first[E] = at;
    }
    __syncthreads();
    for (int i = tid; i < n_entries; i += 1024) {
        const int e = ids[i];
        if (e < 0 || e >= E) continue;
        const int place = first[e] + atomicAdd(&counts[e], 1);
        if (place < max_tiles * block) rows_list[place] = i;
    }
}

__global__ void __launch_bounds__(1024)
moe_align_kernel(const int* __restrict__ ids, int n_entries, int E, int block, int* __restrict__ rows_list, int* __restrict__ tile_group,
                 int max_tiles) {
    extern __shared__ int sh[];
    align_entries(ids, n_entries, E, block, rows_list, tile_group, max_tiles, sh);
}

// Both in one launch for steps of at most 1,024 tokens: a thread routes a token, then the workgroup lists the entries.
__global__ void __launch_bounds__(1024)
moe_route_align_kernel(const float* __restrict__ logits, int64_t ld, int n, int E, int top, int* __restrict__ ids, float* __restrict__ weights,
                       int block, int* __restrict__ rows_list, int* __restrict__ tile_group, int max_tiles, int mode, int n_groups, int keep) {
    extern __shared__ int sh[];
    const int t = threadIdx.x;
    if (t < n) route_any(logits + static_cast<int64_t>(t) * ld, E, top, mode, n_groups, keep, ids + static_cast<int64_t>(t) * top, weights + static_cast<int64_t>(t) * top);
    __syncthreads();  // (the ids are read back by other threads of this workgroup)
    align_entries(ids, n * top, E, block, rows_list, tile_group, max_tiles, sh);
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_moe_route(const float* logits, int64_t ld, int n, int n_experts, int top, int* ids, float* weights, int mode, int n_groups,
                               int keep, hipStream_t stream) {
    LIYAB_REQUIRE(logits && ids && weights, "moe_route: null pointer");
    LIYAB_REQUIRE(mode == 0 || (mode == 1 && n_groups >= 1 && n_groups <= kMaxGroups && n_experts % n_groups == 0 && keep >= 1 && keep <= n_groups &&
                                top <= keep * (n_experts / n_groups)),
                  "moe_route: %d of %d groups of %d experts do not hold %d choices (at most %d groups)", keep, n_groups, n_experts, top, kMaxGroups);
    LIYAB_REQUIRE(n >= 0 && n_experts > 0 && top >= 1 && top <= n_experts && top <= kMaxTop && ld >= n_experts,
                  "moe_route: bad sizes n=%d experts=%d top=%d (at most %d choices a token)", n, n_experts, top, kMaxTop);
    if (n == 0) return 0;
    moe_route_kernel<<<(n + 255) / 256, 256, 0, stream>>>(logits, ld, n, n_experts, top, ids, weights, mode, n_groups, keep);
    return check_launch("moe_route");
}

extern "C" int liyab_moe_align(const int* ids, int n_entries, int n_experts, int block, int* rows_list, int* tile_group, int max_tiles,
                               hipStream_t stream) {
    LIYAB_REQUIRE(ids && rows_list && tile_group, "moe_align: null pointer");
    LIYAB_REQUIRE(n_entries >= 0 && n_experts > 0 && n_experts <= 4096 && block > 0, "moe_align: bad sizes (at most 4,096 experts)");
    LIYAB_REQUIRE(static_cast<int64_t>(max_tiles) * block >= static_cast<int64_t>(n_entries) + static_cast<int64_t>(n_entries < n_experts ? n_entries : n_experts) * (block - 1),
                  "moe_align: %d tiles of %d places do not hold %d entries of %d experts", max_tiles, block, n_entries, n_experts);
    if (n_entries == 0) return 0;
    moe_align_kernel<<<1, 1024, (2 * n_experts + 1) * sizeof(int), stream>>>(ids, n_entries, n_experts, block, rows_list, tile_group, max_tiles);
    return check_launch("moe_align");
}

extern "C" int liyab_moe_route_align(const float* logits, int64_t ld, int n, int n_experts, int top, int* ids, float* weights, int block,
                                     int* rows_list, int* tile_group, int max_tiles, int mode, int n_groups, int keep, hipStream_t stream) {
    LIYAB_REQUIRE(n <= 1024, "moe_route_align: %d tokens; one workgroup routes at most 1,024 (moe_route and moe_align take more)", n);
    if (const int rc = liyab_moe_route(logits, ld, 0, n_experts, top, ids, weights, mode, n_groups, keep, stream)) return rc;                    // (the checks of both,
    if (const int rc = liyab_moe_align(ids, 0, n_experts, block, rows_list, tile_group, max_tiles, stream)) return rc;    //  nothing launched)
    LIYAB_REQUIRE(n >= 0 && static_cast<int64_t>(max_tiles) * block >= static_cast<int64_t>(n) * top + static_cast<int64_t>(n * top < n_experts ? n * top : n_experts) * (block - 1),
                  "moe_route_align: %d tiles of %d places do not hold %d entries of %d experts", max_tiles, block, n * top, n_experts);
    if (n == 0) return 0;
    moe_route_align_kernel<<<1, 1024, (2 * n_experts + 1) * sizeof(int), stream>>>(logits, ld, n, n_experts, top, ids, weights, block, rows_list,
                                                                                    tile_group, max_tiles, mode, n_groups, keep);
    return check_launch("moe_route_align");
}
