// Attention in two maps a head that share their values: what stands between the projection and the paged attention kernels,
// and what joins the two maps' results.
//
// liyab_maps_store: from a projection's 32-bit rows [q | k | v] (a query head holds [map 1 | map 2], D values each; a key head
//   the same; a value head V values), every channel first through a causal convolution over time when there is one,
//       y_t = sum_{j < taps} c[:, j] * u_(t - taps + 1 + j)          (zeros before a request's start)
//   whose earlier inputs come from the step's own rows or from the request's history (position p at ring place p % (taps - 1) of
//   its slot, [C] floats a place, kept by liyab_ring_keep after this kernel has run), to
//     queries  [n, 2, H, P]  (map-major, so that each map is a set of H heads of P for the attention kernels),
//     keys of map m in plane m of the pages and values in a third plane, all [pages, G, page_size, P],
//   P >= max(D, V) with zeros behind a head's own entries (zeros add nothing to a score, and nobody reads the values' zeros).
//   Sums are 32-bit, rounded once to the pages' type.
// liyab_maps_join: o = a1 - lam * a2 a head, o / sqrt(mean(o^2 over the head's V) + eps) * out_scale, rounded once.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kMapsMaxTaps = 16;

struct MapsArgs {
    const float* src;   // [n, ld]
    int64_t ld;
    const float* cw;    // [C, taps] or null
    int taps;
    const float* state; // the ring of slot 0; a slot is state_stride floats further
    int64_t state_stride;
    int n_slots;
    void *q_out, *k1, *k2, *vc;
    const int* slots;   // [n]: page * page_size + offset, or outside the pages
    int page_size, num_pages;
    const int *tok_seq, *positions, *seq_starts, *state_slots;
    int H, G, D, V, P;
};

template <typename T>
__global__ void __launch_bounds__(256)
maps_store_kernel(MapsArgs a) {
    const int t = blockIdx.x;
    const int s = a.tok_seq[t], p = a.positions[t];
    const int in_step = t - a.seq_starts[s];
    const int ring = a.taps > 0 ? a.taps - 1 : 0;
    int slot = a.state_slots[s];
    if (slot < 0 || slot >= a.n_slots || a.state == nullptr) slot = -1;
    const int H = a.H, G = a.G, D = a.D, V = a.V, P = a.P;
    const int C = 2 * H * D + 2 * G * D + G * V;
    const float* src[kMapsMaxTaps];  // the row m back, or null
#pragma unroll
    for (int m = 1; m < kMapsMaxTaps; ++m) {
        src[m] = nullptr;
        if (m <= ring && p - m >= 0) {
            if (m <= in_step) src[m] = a.src + static_cast<int64_t>(t - m) * a.ld;
            else if (slot >= 0) src[m] = a.state + static_cast<int64_t>(slot) * a.state_stride + static_cast<int64_t>((p - m) % ring) * C;
        }
    }
    const float* row = a.src + static_cast<int64_t>(t) * a.ld;
    const int cache_slot = a.slots[t];
    const bool cached = cache_slot >= 0 && cache_slot < a.num_pages * a.page_size;
    const int page = cached ? cache_slot / a.page_size : 0, off = cached ? cache_slot % a.page_size : 0;
    const int nq = 2 * H * P, nk = 2 * G * P, nv = G * P;
    for (int e = threadIdx.x; e < nq + nk + nv; e += 256) {
        int c = -1;  // the projection's channel this element holds, or none (padding)
        T* dst = nullptr;
        if (e < nq) {
            const int m = e / (H * P), h = (e / P) % H, i = e % P;
            if (i < D) c = h * 2 * D + m * D + i;
            dst = static_cast<T*>(a.q_out) + static_cast<int64_t>(t) * nq + e;
        } else if (e < nq + nk) {
            const int f = e - nq;
            const int m = f / (G * P), g = (f / P) % G, i = f % P;
            if (i < D) c = 2 * H * D + g * 2 * D + m * D + i;
            if (cached) dst = static_cast<T*>(m == 0 ? a.k1 : a.k2) + ((static_cast<int64_t>(page) * G + g) * a.page_size + off) * P + i;
        } else {
            const int f = e - nq - nk;
            const int g = f / P, i = f % P;
            if (i < V) c = 2 * H * D + 2 * G * D + g * V + i;
            if (cached) dst = static_cast<T*>(a.vc) + ((static_cast<int64_t>(page) * G + g) * a.page_size + off) * P + i;
        }
        if (dst == nullptr) continue;
        float acc = 0.0f;
        if (c >= 0) {
            if (a.cw == nullptr) acc = row[c];
            else {
                const float* w = a.cw + static_cast<int64_t>(c) * a.taps;
                acc = w[a.taps - 1] * row[c];
#pragma unroll
                for (int m = 1; m < kMapsMaxTaps; ++m)
                    if (m <= ring && src[m] != nullptr) acc += w[a.taps - 1 - m] * src[m][c];
            }
        }
        *dst = from_float<T>(acc);
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
maps_join_kernel(T* __restrict__ out, const T* __restrict__ a1, const T* __restrict__ a2, int64_t lda, float lam, float eps, float out_scale,
                 int n, int H, int V, int P) {
    const int item = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (item >= n * H) return;
    const int t = item / H, h = item % H;
    const T* r1 = a1 + static_cast<int64_t>(t) * lda + h * P;
    const T* r2 = a2 + static_cast<int64_t>(t) * lda + h * P;
    float ss = 0.0f;
    for (int i = lane; i < V; i += kWave) {
        const float o = to_float<T>(r1[i]) - lam * to_float<T>(r2[i]);
        ss += o * o;
    }
    const float scale = out_scale / sqrtf(wave_sum(ss) / static_cast<float>(V) + eps);
    for (int i = lane; i < V; i += kWave) {
        const float o = to_float<T>(r1[i]) - lam * to_float<T>(r2[i]);
        out[(static_cast<int64_t>(t) * H + h) * V + i] = from_float<T>(o * scale);
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_maps_store(const float* src, int64_t ld, const float* cw, int taps, const float* state, int64_t state_stride, int n_slots,
                                void* q_out, void* k1, void* k2, void* vc, int dtype, const int* slots, int page_size, int num_pages,
                                const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots, int n, int H, int G,
                                int D, int V, int P, hipStream_t stream) {
    LIYAB_REQUIRE(src && q_out && k1 && k2 && vc && slots && tok_seq && positions && seq_starts && state_slots, "maps_store: null pointer");
    LIYAB_REQUIRE(n >= 0 && H > 0 && G > 0 && D > 0 && V > 0 && P >= D && P >= V && page_size > 0 && num_pages > 0, "maps_store: bad sizes");
    const int64_t C = 2LL * H * D + 2LL * G * D + 1LL * G * V;
    LIYAB_REQUIRE(ld >= C, "maps_store: rows of %lld floats hold no %lld channels", static_cast<long long>(ld), static_cast<long long>(C));
    LIYAB_REQUIRE(cw == nullptr ? taps == 0 : (taps >= 1 && taps <= kMapsMaxTaps), "maps_store: %d taps; 1 to %d are taken", taps, kMapsMaxTaps);
    LIYAB_REQUIRE(taps <= 1 || (state != nullptr && n_slots > 0 && state_stride >= (taps - 1) * C), "maps_store: %d taps need the requests' history", taps);
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "maps_store: unknown dtype %d", dtype);
    if (n == 0) return 0;
    MapsArgs a{src, ld, cw, taps, state, state_stride, n_slots, q_out, k1, k2, vc, slots, page_size, num_pages, tok_seq, positions, seq_starts,
               state_slots, H, G, D, V, P};
    if (dtype == kF32) maps_store_kernel<float><<<n, 256, 0, stream>>>(a);
    else maps_store_kernel<bf16_t><<<n, 256, 0, stream>>>(a);
    return check_launch("maps_store");
}

extern "C" int liyab_maps_join(void* out, const void* a1, const void* a2, int64_t lda, int dtype, float lam, float eps, float out_scale, int n,
                               int H, int V, int P, hipStream_t stream) {
    LIYAB_REQUIRE(out && a1 && a2, "maps_join: null pointer");
    LIYAB_REQUIRE(n >= 0 && H > 0 && V > 0 && P >= V && lda >= static_cast<int64_t>(H) * P, "maps_join: bad sizes");
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "maps_join: unknown dtype %d", dtype);
    if (n == 0) return 0;
    const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(n) * H + 3) / 4);
    if (dtype == kF32)
        maps_join_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(a1), static_cast<const float*>(a2), lda, lam, eps,
                                                          out_scale, n, H, V, P);
    else
        maps_join_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), static_cast<const bf16_t*>(a1), static_cast<const bf16_t*>(a2), lda, lam,
                                                           eps, out_scale, n, H, V, P);
    return check_launch("maps_join");
}
