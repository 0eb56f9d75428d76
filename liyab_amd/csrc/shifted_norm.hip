// What a block of two parallel sublayers does to the stream before they read it, and small row kernels around them.
//
// liyab_norm_shift: one pass over a row of the 32-bit stream gives every sublayer its input:
//   h_s = x / sqrt(mean(x^2) + eps) * (w_s + offset),            s = 0 .. S - 1 (the sublayers share the root mean square)
//   out_s[t] = h_s[t] + sum_{j < taps} c_s[j, :] * h_s[t - taps + 1 + j]     (zeros before a request's start; no c: out = h;
//                                                                              c is [S, taps, d]: a tap's channels side by side)
// A source row inside the step's portion is normalised again by the workgroup that needs it (the same arithmetic in the
// same order as its own workgroup's, so the same bits); an earlier one is read, already normalised, from the request's
// history: position p at ring place p % (taps - 1) of state[slot], each place holding [S, d] floats. `hbuf` [n, S * d]
// gets h itself for liyab_ring_keep, which runs after every kernel that reads the ring; with `keep_single`, a request that
// brings one token keeps its row here (a step of single tokens needs no keeper). Everything is 32-bit; the result is rounded
// once to the output type. Rows behind the step's tokens (position 0 of the first request) read no history.
//
// liyab_ring_keep: the last `ring` rows of each request in the step, columns [0, width) of src, go to its history.
// liyab_normed_powers: out = c1 N(z) + c2 N(z^2) + c3 N(z^3) + c4, N(v) = v / sqrt(mean(v^2) + eps) over a row of z.
// liyab_softcap: p <- cap * tanh(p / cap) in place.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kShiftThreads = 256;
constexpr int kShiftMaxTaps = 16;
constexpr int kShiftMaxSub = 2;

// sums of `COUNT` values over a workgroup of kShiftThreads, every thread getting all of them; red: [COUNT][waves]
template <int COUNT>
__device__ __forceinline__ void block_sums(float (&v)[COUNT], float* red) {
    constexpr int WAVES = kShiftThreads / kWave;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
    for (int i = 0; i < COUNT; ++i) v[i] = wave_sum(v[i]);
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < COUNT; ++i) red[i * WAVES + wave] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < COUNT; ++i) {
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) total += red[i * WAVES + w];
        v[i] = total;
    }
}

template <typename T, int MAXT>
__global__ void __launch_bounds__(kShiftThreads)
norm_shift_kernel(T* __restrict__ out, float* __restrict__ hbuf, const float* __restrict__ x, const float* __restrict__ w, float offset, float eps,
                  const float* __restrict__ cw, int taps, float* state, int64_t state_stride, int n_slots,
                  const int* __restrict__ tok_seq, const int* __restrict__ positions, const int* __restrict__ seq_starts,
                  const int* __restrict__ state_slots, int n, int d, int S, int keep_single) {
    __shared__ float red[MAXT * (kShiftThreads / kWave)];
    const int t = blockIdx.x;
    const int s = tok_seq[t], p = positions[t];
    const int in_step = t - seq_starts[s];
    const int ring = taps > 0 ? taps - 1 : 0;
    int slot = state_slots[s];
    if (slot < 0 || slot >= n_slots || state == nullptr) slot = -1;
    // source m rows back: 1 = a row of the step, 2 = a place of the ring, 0 = nothing
    int kind[MAXT];
    float ss[MAXT];
#pragma unroll
    for (int m = 0; m < MAXT; ++m) {
        kind[m] = 0;
        if (m == 0) kind[m] = 1;
        else if (m <= ring && p - m >= 0) kind[m] = m <= in_step ? 1 : (slot >= 0 ? 2 : 0);
        ss[m] = 0.0f;
    }
    for (int i = threadIdx.x; i < d; i += kShiftThreads) {
#pragma unroll
        for (int m = 0; m < MAXT; ++m) {
            const float v = x[static_cast<int64_t>(kind[m] == 1 ? t - m : t) * d + i];
            ss[m] += kind[m] == 1 ? v * v : 0.0f;
        }
    }
    block_sums<MAXT>(ss, red);
    float scale[MAXT];
#pragma unroll
    for (int m = 0; m < MAXT; ++m) scale[m] = 1.0f / sqrtf(ss[m] / static_cast<float>(d) + eps);
    const int64_t place = static_cast<int64_t>(S) * d;
    float* hist = slot >= 0 ? state + static_cast<int64_t>(slot) * state_stride : nullptr;
    // a request that brings one token: its row takes its place in the ring here (the place of the oldest row, which the same
    // thread has just read), and no keeper runs behind this kernel
    const bool keep_own = keep_single != 0 && ring > 0 && slot >= 0 && seq_starts[s + 1] - seq_starts[s] == 1;
    for (int i = threadIdx.x; i < d; i += kShiftThreads) {
        float xs[MAXT];
#pragma unroll
        for (int m = 0; m < MAXT; ++m) xs[m] = kind[m] == 1 ? x[static_cast<int64_t>(t - m) * d + i] * scale[m] : 0.0f;
        for (int sub = 0; sub < S; ++sub) {
            const float wi = w[static_cast<int64_t>(sub) * d + i] + offset;
            const float h0 = xs[0] * wi;
            float acc = h0;
            if (cw != nullptr) {
                const float* c = cw + (static_cast<int64_t>(sub) * taps + taps - 1) * d + i;  // (the newest tap; tap j of a channel lies d floats further a tap)
                acc += c[0] * h0;
#pragma unroll
                for (int m = 1; m < MAXT; ++m) {
                    if (kind[m] == 1) acc += c[-static_cast<int64_t>(m) * d] * (xs[m] * wi);
                    else if (kind[m] == 2) acc += c[-static_cast<int64_t>(m) * d] * hist[((p - m) % ring) * place + static_cast<int64_t>(sub) * d + i];
                }
            }
            out[(static_cast<int64_t>(sub) * n + t) * d + i] = from_float<T>(acc);
            if (hbuf != nullptr) hbuf[static_cast<int64_t>(t) * place + static_cast<int64_t>(sub) * d + i] = h0;
            if (keep_own) hist[(p % ring) * place + static_cast<int64_t>(sub) * d + i] = h0;
        }
    }
}

// The same for widths that are multiples of four and rows that start at multiples of 16 bytes: a thread takes four channels side
// by side, so that a row of up to 1,024 channels is one trip to memory a pass, 16 bytes a load, and both sublayers' loads are on
// their way together. A row's sum of squares is added up in the same order whichever workgroup needs it.
template <typename T, int MAXT>
__global__ void __launch_bounds__(kShiftThreads)
norm_shift_vec_kernel(T* __restrict__ out, float* __restrict__ hbuf, const float* __restrict__ x, const float* __restrict__ w, float offset, float eps,
                      const float* __restrict__ cw, int taps, float* state, int64_t state_stride, int n_slots,
                      const int* __restrict__ tok_seq, const int* __restrict__ positions, const int* __restrict__ seq_starts,
                      const int* __restrict__ state_slots, int n, int d, int S, int keep_single) {
    __shared__ float red[MAXT * (kShiftThreads / kWave)];
    const int t = blockIdx.x;
    const int s = tok_seq[t], p = positions[t];
    const int in_step = t - seq_starts[s];
    const int ring = taps > 0 ? taps - 1 : 0;
    int slot = state_slots[s];
    if (slot < 0 || slot >= n_slots || state == nullptr) slot = -1;
    int kind[MAXT];  // source m rows back: 1 = a row of the step, 2 = a place of the ring, 0 = nothing
    float ss[MAXT];
#pragma unroll
    for (int m = 0; m < MAXT; ++m) {
        kind[m] = 0;
        if (m == 0) kind[m] = 1;
        else if (m <= ring && p - m >= 0) kind[m] = m <= in_step ? 1 : (slot >= 0 ? 2 : 0);
        ss[m] = 0.0f;
    }
    for (int i = threadIdx.x * 4; i < d; i += kShiftThreads * 4) {
#pragma unroll
        for (int m = 0; m < MAXT; ++m) {
            if (kind[m] == 1) {
                const f32x4_t v = *reinterpret_cast<const f32x4_t*>(x + static_cast<int64_t>(t - m) * d + i);
                ss[m] += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
            }
        }
    }
    block_sums<MAXT>(ss, red);
    float scale[MAXT];
#pragma unroll
    for (int m = 0; m < MAXT; ++m) scale[m] = 1.0f / sqrtf(ss[m] / static_cast<float>(d) + eps);
    const int64_t place = static_cast<int64_t>(S) * d;
    float* hist = slot >= 0 ? state + static_cast<int64_t>(slot) * state_stride : nullptr;
    // a request that brings one token: its row takes its place in the ring here (the place of the oldest row, which the same
    // thread has just read), and no keeper runs behind this kernel
    const bool keep_own = keep_single != 0 && ring > 0 && slot >= 0 && seq_starts[s + 1] - seq_starts[s] == 1;
    for (int i = threadIdx.x * 4; i < d; i += kShiftThreads * 4) {
        f32x4_t xs[MAXT];
#pragma unroll
        for (int m = 0; m < MAXT; ++m) {
            xs[m] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            if (kind[m] == 1) xs[m] = *reinterpret_cast<const f32x4_t*>(x + static_cast<int64_t>(t - m) * d + i) * scale[m];
        }
#pragma unroll
        for (int sub = 0; sub < kShiftMaxSub; ++sub) {
            if (sub >= S) break;
            const f32x4_t wi = *reinterpret_cast<const f32x4_t*>(w + static_cast<int64_t>(sub) * d + i) + offset;
            const f32x4_t h0 = xs[0] * wi;
            float acc[4] = {h0[0], h0[1], h0[2], h0[3]};
            if (cw != nullptr) {
                const float* c = cw + (static_cast<int64_t>(sub) * taps + taps - 1) * d + i;  // (the newest tap of four channels side by side)
                const f32x4_t c0 = *reinterpret_cast<const f32x4_t*>(c);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += c0[e] * h0[e];
#pragma unroll
                for (int m = 1; m < MAXT; ++m) {
                    if (kind[m] == 0) continue;
                    const f32x4_t cm = *reinterpret_cast<const f32x4_t*>(c - static_cast<int64_t>(m) * d);
                    if (kind[m] == 1) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[e] += cm[e] * (xs[m][e] * wi[e]);
                    } else {
                        const f32x4_t hv = *reinterpret_cast<const f32x4_t*>(hist + ((p - m) % ring) * place + static_cast<int64_t>(sub) * d + i);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[e] += cm[e] * hv[e];
                    }
                }
            }
            store4<T>(out + (static_cast<int64_t>(sub) * n + t) * d + i, acc);
            if (hbuf != nullptr) *reinterpret_cast<f32x4_t*>(hbuf + static_cast<int64_t>(t) * place + static_cast<int64_t>(sub) * d + i) = h0;
            if (keep_own) *reinterpret_cast<f32x4_t*>(hist + (p % ring) * place + static_cast<int64_t>(sub) * d + i) = h0;
        }
    }
}

__global__ void __launch_bounds__(256)
ring_keep_kernel(float* __restrict__ state, int64_t state_stride, int ring, int n_slots, const float* __restrict__ src, int64_t ld, int width,
                 const int* __restrict__ tok_seq, const int* __restrict__ positions, const int* __restrict__ context_lens,
                 const int* __restrict__ state_slots, const int* __restrict__ n_real) {
    const int t = blockIdx.x;
    if (t >= *n_real) return;
    const int s = tok_seq[t], p = positions[t], slot = state_slots[s];
    if (p < context_lens[s] - ring || slot < 0 || slot >= n_slots) return;
    float* dst = state + static_cast<int64_t>(slot) * state_stride + static_cast<int64_t>(p % ring) * width;
    const float* row = src + static_cast<int64_t>(t) * ld;
    for (int i = threadIdx.x; i < width; i += 256) dst[i] = row[i];
}

template <typename T>
__global__ void __launch_bounds__(kShiftThreads)
normed_powers_kernel(T* __restrict__ out, const float* __restrict__ z, int64_t ld, int ff, const float* __restrict__ coef, float eps) {
    __shared__ float red[3 * (kShiftThreads / kWave)];
    const float* row = z + static_cast<int64_t>(blockIdx.x) * ld;
    float ss[3] = {0.0f, 0.0f, 0.0f};
    for (int i = threadIdx.x; i < ff; i += kShiftThreads) {
        const float v = row[i], v2 = v * v;
        ss[0] += v2;
        ss[1] += v2 * v2;
        ss[2] += v2 * v2 * v2;
    }
    block_sums<3>(ss, red);
    const float inv = 1.0f / static_cast<float>(ff);
    const float c1 = coef[0] / sqrtf(ss[0] * inv + eps), c2 = coef[1] / sqrtf(ss[1] * inv + eps), c3 = coef[2] / sqrtf(ss[2] * inv + eps);
    const float c4 = coef[3];
    T* o = out + static_cast<int64_t>(blockIdx.x) * ff;
    for (int i = threadIdx.x; i < ff; i += kShiftThreads) {
        const float v = row[i], v2 = v * v;
        o[i] = from_float<T>(c1 * v + c2 * v2 + c3 * (v2 * v) + c4);
    }
}

__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ p, float cap, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) p[i] = cap * tanhf(p[i] / cap);
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_norm_shift(void* out, int out_dtype, float* hbuf, const float* x, const float* w, float offset, float eps, const float* cw,
                                int taps, float* state, int64_t state_stride, int n_slots, const int* tok_seq, const int* positions,
                                const int* seq_starts, const int* state_slots, int n, int d, int S, int keep_single, hipStream_t stream) {
    LIYAB_REQUIRE(out && x && w && tok_seq && positions && seq_starts && state_slots, "norm_shift: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0 && S >= 1 && S <= kShiftMaxSub, "norm_shift: bad sizes n=%d d=%d sublayers=%d", n, d, S);
    LIYAB_REQUIRE(cw == nullptr ? taps == 0 : (taps >= 1 && taps <= kShiftMaxTaps), "norm_shift: %d taps; 1 to %d are taken", taps, kShiftMaxTaps);
    LIYAB_REQUIRE(taps <= 1 || (state != nullptr && n_slots > 0 && state_stride >= static_cast<int64_t>(taps - 1) * S * d),
                  "norm_shift: %d taps need the requests' history", taps);
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "norm_shift: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    const auto at16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    const bool vec = d % 4 == 0 && at16(out) && at16(hbuf) && at16(x) && at16(w) && at16(cw) && (taps <= 1 || (at16(state) && state_stride % 4 == 0));
#define LIYAB_SHIFT(T, MAXT)                                                                                                                  \
    do { if (vec)                                                                                                                             \
        norm_shift_vec_kernel<T, MAXT><<<n, kShiftThreads, 0, stream>>>(static_cast<T*>(out), hbuf, x, w, offset, eps, cw, taps, state,      \
                                                                          state_stride, n_slots, tok_seq, positions, seq_starts, state_slots, \
                                                                          n, d, S, keep_single);                                              \
    else                                                                                                                                      \
        norm_shift_kernel<T, MAXT><<<n, kShiftThreads, 0, stream>>>(static_cast<T*>(out), hbuf, x, w, offset, eps, cw, taps, state,          \
                                                                      state_stride, n_slots, tok_seq, positions, seq_starts, state_slots, n, \
                                                                      d, S, keep_single); } while (0)
    if (out_dtype == kF32) {
        if (taps <= 1) LIYAB_SHIFT(float, 1);
        else if (taps <= 4) LIYAB_SHIFT(float, 4);
        else LIYAB_SHIFT(float, kShiftMaxTaps);
    } else {
        if (taps <= 1) LIYAB_SHIFT(bf16_t, 1);
        else if (taps <= 4) LIYAB_SHIFT(bf16_t, 4);
        else LIYAB_SHIFT(bf16_t, kShiftMaxTaps);
    }
#undef LIYAB_SHIFT
    return check_launch("norm_shift");
}

extern "C" int liyab_ring_keep(float* state, int64_t state_stride, int ring, int n_slots, const float* src, int64_t ld, int width,
                               const int* tok_seq, const int* positions, const int* context_lens, const int* state_slots, const int* n_real,
                               int n, hipStream_t stream) {
    LIYAB_REQUIRE(state && src && tok_seq && positions && context_lens && state_slots && n_real, "ring_keep: null pointer");
    LIYAB_REQUIRE(n >= 0 && width > 0 && ld >= width && ring > 0 && n_slots > 0 && state_stride >= static_cast<int64_t>(ring) * width,
                  "ring_keep: bad sizes");
    if (n == 0) return 0;
    ring_keep_kernel<<<n, 256, 0, stream>>>(state, state_stride, ring, n_slots, src, ld, width, tok_seq, positions, context_lens, state_slots, n_real);
    return check_launch("ring_keep");
}

extern "C" int liyab_normed_powers(void* out, int out_dtype, const float* z, int64_t ld, int n, int ff, const float* coef, float eps,
                                   hipStream_t stream) {
    LIYAB_REQUIRE(out && z && coef, "normed_powers: null pointer");
    LIYAB_REQUIRE(n >= 0 && ff > 0 && ld >= ff, "normed_powers: bad sizes n=%d ff=%d", n, ff);
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "normed_powers: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    if (out_dtype == kF32) normed_powers_kernel<float><<<n, kShiftThreads, 0, stream>>>(static_cast<float*>(out), z, ld, ff, coef, eps);
    else normed_powers_kernel<bf16_t><<<n, kShiftThreads, 0, stream>>>(static_cast<bf16_t*>(out), z, ld, ff, coef, eps);
    return check_launch("normed_powers");
}

extern "C" int liyab_softcap(float* p, float cap, int64_t n, hipStream_t stream) {
    LIYAB_REQUIRE(p != nullptr && n >= 0 && cap > 0.0f, "softcap: bad operands");
    if (n == 0) return 0;
    softcap_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(p, cap, n);
    return check_launch("softcap");
}
