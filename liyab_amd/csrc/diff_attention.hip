// Attention in two maps a head that share their values: what stands between the projection and the paged attention kernels,
// and what joins the two maps' results.
//
// liyab_maps_store: from a projection's 32-bit rows [q | k | v] (a query head holds [map 1 | map 2], D values each; a key head
//   the same; a value head V values), every channel first through a causal convolution over time when there is one,
//       y_t = sum_{j < taps} c[j, :] * u_(t - taps + 1 + j)          (zeros before a request's start; c is [taps, C])
//   whose earlier inputs come from the step's own rows or from the request's history (position p at ring place p % (taps - 1) of
//   its slot, [C] floats a place, kept by liyab_ring_keep after this kernel has run, or, with `keep_single`, by this kernel for a
//   request that brings one token), to
//     queries  [n, 2, H, P]  (map-major, so that each map is a set of H heads of P for the attention kernels),
//     keys of map m in plane m of the pages and values in a third plane, all [pages, G, page_size, P],
//   P >= max(D, V) with zeros behind a head's own entries (zeros add nothing to a score, and nobody reads the values' zeros).
//   Sums are 32-bit, rounded once to the pages' type.
// liyab_maps_join: o = a1 - lam * a2 a head, o / sqrt(mean(o^2 over the head's V) + eps) * out_scale, rounded once.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kMapsMaxTaps = 16;
constexpr int kMapsUnits = 8;  // units a workgroup: two a wave

struct MapsArgs {
    const float* src;   // [n, ld]
    int64_t ld;
    const float* cw;    // [taps, C] or null
    int taps;
    float* state;       // the ring of slot 0; a slot is state_stride floats further
    int keep_single;    // a request that brings one token keeps its projected row in the ring here (no keeper behind this kernel)
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
    float* keep = (a.keep_single != 0 && ring > 0 && slot >= 0 && a.seq_starts[s + 1] - a.seq_starts[s] == 1)
                      ? a.state + static_cast<int64_t>(slot) * a.state_stride + static_cast<int64_t>(p % ring) * C : nullptr;
    const int cache_slot = a.slots[t];
    const bool cached = cache_slot >= 0 && cache_slot < a.num_pages * a.page_size;
    const int page = cached ? cache_slot / a.page_size : 0, off = cached ? cache_slot % a.page_size : 0;
    const int nq = 2 * H * P;
    // a unit: one head's P entries of one destination (queries of a map, keys of a map, values); a wave a unit, kMapsUnits a
    // workgroup, so that a step of few rows still spreads over the chip
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
    const int n_units = 2 * H + 3 * G;
    const int unit_end = min(n_units, static_cast<int>(blockIdx.y + 1) * kMapsUnits);
    for (int unit = blockIdx.y * kMapsUnits + wave; unit < unit_end; unit += 256 / kWave) {
        int c0, width;  // the projection's first channel of this unit and how many it has (the rest of P is padding)
        T* dst = nullptr;
        if (unit < 2 * H) {
            const int m = unit / H, h = unit % H;
            c0 = h * 2 * D + m * D;
            width = D;
            dst = static_cast<T*>(a.q_out) + static_cast<int64_t>(t) * nq + static_cast<int64_t>(unit) * P;
        } else if (unit < 2 * H + 2 * G) {
            const int f = unit - 2 * H;
            const int m = f / G, g = f % G;
            c0 = 2 * H * D + g * 2 * D + m * D;
            width = D;
            if (cached) dst = static_cast<T*>(m == 0 ? a.k1 : a.k2) + ((static_cast<int64_t>(page) * G + g) * a.page_size + off) * P;
        } else {
            const int g = unit - 2 * H - 2 * G;
            c0 = 2 * H * D + 2 * G * D + g * V;
            width = V;
            if (cached) dst = static_cast<T*>(a.vc) + ((static_cast<int64_t>(page) * G + g) * a.page_size + off) * P;
        }
        if (dst == nullptr && keep == nullptr) continue;
        for (int i = lane; i < P; i += kWave) {
            float acc = 0.0f;
            if (i < width) {
                const int c = c0 + i;
                const float x0 = row[c];
                if (a.cw == nullptr) acc = x0;
                else {
                    const float* w = a.cw + static_cast<int64_t>(a.taps - 1) * C + c;  // (the newest tap; a tap's channels lie side by side)
                    acc = w[0] * x0;
#pragma unroll
                    for (int m = 1; m < kMapsMaxTaps; ++m)
                        if (m <= ring && src[m] != nullptr) acc += w[-static_cast<int64_t>(m) * C] * src[m][c];
                }
                if (keep != nullptr) keep[c] = x0;  // (the oldest row's place: this thread has just read it)
            }
            if (dst != nullptr) dst[i] = from_float<T>(acc);
        }
    }
}

// The same for head sizes that are multiples of four (and rows that start at multiples of 16 bytes): a thread takes four channels
// side by side of one row, a workgroup 1,024 of a row's channels, so that every load is 16 bytes wide and all of a thread's
// loads are on their way together; the zeros behind the narrower heads are written after that.
template <typename T>
__global__ void __launch_bounds__(256)
maps_store_vec_kernel(MapsArgs a) {
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    const int t = blockIdx.x;
    const int s = a.tok_seq[t], p = a.positions[t];
    const int in_step = t - a.seq_starts[s];
    const int ring = a.taps > 0 ? a.taps - 1 : 0;
    int slot = a.state_slots[s];
    if (slot < 0 || slot >= a.n_slots || a.state == nullptr) slot = -1;
    const int H = a.H, G = a.G, D = a.D, V = a.V, P = a.P;
    const int QC = 2 * H * D, KC = 2 * G * D, C = QC + KC + G * V;
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
    float* keep = (a.keep_single != 0 && ring > 0 && slot >= 0 && a.seq_starts[s + 1] - a.seq_starts[s] == 1)
                      ? a.state + static_cast<int64_t>(slot) * a.state_stride + static_cast<int64_t>(p % ring) * C : nullptr;
    const int cache_slot = a.slots[t];
    const bool cached = cache_slot >= 0 && cache_slot < a.num_pages * a.page_size;
    const int page = cached ? cache_slot / a.page_size : 0, off = cached ? cache_slot % a.page_size : 0;
    const int64_t nq = 2LL * H * P;
    T* const q_row = static_cast<T*>(a.q_out) + static_cast<int64_t>(t) * nq;
    auto paged = [&](void* plane, int g) { return static_cast<T*>(plane) + ((static_cast<int64_t>(page) * G + g) * a.page_size + off) * P; };
    const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c < C) {
        T* dst = nullptr;
        if (c < QC) {
            const int h = c / (2 * D), r = c % (2 * D);
            dst = q_row + static_cast<int64_t>((r / D) * H + h) * P + r % D;
        } else if (c < QC + KC) {
            const int f = c - QC;
            const int g = f / (2 * D), r = f % (2 * D);
            if (cached) dst = paged(r / D == 0 ? a.k1 : a.k2, g) + r % D;
        } else {
            const int f = c - QC - KC;
            if (cached) dst = paged(a.vc, f / V) + f % V;
        }
        if (dst != nullptr || keep != nullptr) {
            const f32x4 x0 = *reinterpret_cast<const f32x4*>(row + c);
            float acc[4] = {x0[0], x0[1], x0[2], x0[3]};
            if (a.cw != nullptr) {
                const float* w = a.cw + static_cast<int64_t>(a.taps - 1) * C + c;  // (the newest tap of four channels side by side)
                const f32x4 w0 = *reinterpret_cast<const f32x4*>(w);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] *= w0[e];
#pragma unroll
                for (int m = 1; m < kMapsMaxTaps; ++m) {
                    if (m <= ring && src[m] != nullptr) {
                        const f32x4 xm = *reinterpret_cast<const f32x4*>(src[m] + c), wm = *reinterpret_cast<const f32x4*>(w - static_cast<int64_t>(m) * C);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[e] += wm[e] * xm[e];
                    }
                }
            }
            if (keep != nullptr) *reinterpret_cast<f32x4*>(keep + c) = x0;  // (the oldest row's place: this thread has just read it)
            if (dst != nullptr) store4<T>(dst, acc);
        }
    }
    // zeros behind the heads' own entries
    const int pad_k = P - D, pad_v = P - V;
    const int n_qpad = 2 * H * pad_k, n_kpad = 2 * G * pad_k, n_vpad = G * pad_v;
    for (int e = blockIdx.y * 256 + threadIdx.x; e < n_qpad + n_kpad + n_vpad; e += gridDim.y * 256) {
        T* dst = nullptr;
        if (e < n_qpad) dst = q_row + static_cast<int64_t>(e / pad_k) * P + D + e % pad_k;
        else if (e < n_qpad + n_kpad) {
            const int f = e - n_qpad;
            const int unit = f / pad_k;
            if (cached) dst = paged(unit / G == 0 ? a.k1 : a.k2, unit % G) + D + f % pad_k;
        } else {
            const int f = e - n_qpad - n_kpad;
            if (cached) dst = paged(a.vc, f / pad_v) + V + f % pad_v;
        }
        if (dst != nullptr) *dst = from_float<T>(0.0f);
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

extern "C" int liyab_maps_store(const float* src, int64_t ld, const float* cw, int taps, float* state, int64_t state_stride, int n_slots,
                                void* q_out, void* k1, void* k2, void* vc, int dtype, const int* slots, int page_size, int num_pages,
                                const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots, int n, int H, int G,
                                int D, int V, int P, int keep_single, hipStream_t stream) {
    LIYAB_REQUIRE(src && q_out && k1 && k2 && vc && slots && tok_seq && positions && seq_starts && state_slots, "maps_store: null pointer");
    LIYAB_REQUIRE(n >= 0 && H > 0 && G > 0 && D > 0 && V > 0 && P >= D && P >= V && page_size > 0 && num_pages > 0, "maps_store: bad sizes");
    const int64_t C = 2LL * H * D + 2LL * G * D + 1LL * G * V;
    LIYAB_REQUIRE(ld >= C, "maps_store: rows of %lld floats hold no %lld channels", static_cast<long long>(ld), static_cast<long long>(C));
    LIYAB_REQUIRE(cw == nullptr ? taps == 0 : (taps >= 1 && taps <= kMapsMaxTaps), "maps_store: %d taps; 1 to %d are taken", taps, kMapsMaxTaps);
    LIYAB_REQUIRE(taps <= 1 || (state != nullptr && n_slots > 0 && state_stride >= (taps - 1) * C), "maps_store: %d taps need the requests' history", taps);
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "maps_store: unknown dtype %d", dtype);
    if (n == 0) return 0;
    MapsArgs a{src, ld, cw, taps, state, keep_single, state_stride, n_slots, q_out, k1, k2, vc, slots, page_size, num_pages, tok_seq, positions, seq_starts,
               state_slots, H, G, D, V, P};
    const auto at16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    if (D % 4 == 0 && V % 4 == 0 && ld % 4 == 0 && at16(src) && at16(cw) && at16(q_out) && at16(k1) && at16(k2) && at16(vc) &&
        (state == nullptr || (at16(state) && state_stride % 4 == 0))) {
        const dim3 grid(n, static_cast<unsigned>((C / 4 + 255) / 256));
        if (dtype == kF32) maps_store_vec_kernel<float><<<grid, 256, 0, stream>>>(a);
        else maps_store_vec_kernel<bf16_t><<<grid, 256, 0, stream>>>(a);
        return check_launch("maps_store");
    }
    const dim3 grid(n, (2 * H + 3 * G + kMapsUnits - 1) / kMapsUnits);
    if (dtype == kF32) maps_store_kernel<float><<<grid, 256, 0, stream>>>(a);
    else maps_store_kernel<bf16_t><<<grid, 256, 0, stream>>>(a);
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
