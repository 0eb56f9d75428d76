// Root-mean-square norms over rows of the 32-bit residual stream.
//
// liyab_rmsnorm: y = x / sqrt(mean(x^2) + eps) * w, the epsilon inside the root; `rows`, when
// given, gathers (the final norm runs on the wanted rows only). Sums and the scaling are 32-bit,
// the result is rounded once to the output type.
//
// liyab_gated_norm_add: the residual update of a block whose norm stands behind its sublayer:
//   s = (y_0 + ... + y_{n_sum-1}) * sigmoid(g),   x += w * s / sqrt(mean(s^2) + eps)
// y: the sublayer's 32-bit result, one row a token or n_sum consecutive rows a token that are
// added in their order (a routed feed-forward leaves one row for each expert a token took);
// without `normalize` the sum is added as it is (x += s);
// g: the gate's 32-bit logits (a pointer and a row stride, so that they may be columns of a wider
// product), or none. The new row may also be written rounded to the compute type for the next
// product (`cast_out`), or, with `next_w`, what the next sublayer reads of it: the new row's own root-mean-square norm under that
// weight and `next_eps` (a block with a norm before its sublayers as well as behind them). Before a row is updated it may be kept as the request's input history of
// a causal convolution over time: `state` [slots, ring, d] holds position p at ring place p % ring,
// and the last `ring` rows of each request in the step are the ones that a later step reads.
#include "common.h"
#include "launchers.h"

namespace liyab {

template <int THREADS>
__device__ __forceinline__ float rms_block_sum(float v, float* red) {
    constexpr int WAVES = THREADS / kWave;
    v = wave_sum(v);
    if constexpr (WAVES == 1) return v;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    __syncthreads();  // red may still be read from a previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) total += red[i];
    return total;
}

template <typename T, int THREADS>
__global__ void __launch_bounds__(THREADS)
rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w, const int* __restrict__ rows,
               int d, float eps) {
    __shared__ float red[THREADS / kWave];
    const int r = blockIdx.x;
    const int64_t src = rows != nullptr ? rows[r] : r;
    const float* xr = x + src * d;
    T* o = out + static_cast<int64_t>(r) * d;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < d; i += THREADS) ss += xr[i] * xr[i];
    const float scale = 1.0f / sqrtf(rms_block_sum<THREADS>(ss, red) / static_cast<float>(d) + eps);
    for (int i = threadIdx.x; i < d; i += THREADS) {
        float v = xr[i] * scale;
        if (w != nullptr) v *= w[i];
        o[i] = from_float<T>(v);
    }
}

struct KeepRows {
    float* state;  // [n_slots, ring, d] or null
    int ring, n_slots;
    const int* tok_seq;
    const int* positions;
    const int* context_lens;
    const int* state_slots;
    const int* n_real;  // the number of rows that belong to a request (rows behind them are padding)
};

__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }

// MAXV values a thread are held in registers between the two passes (d <= THREADS * MAXV); wider
// rows are read again.
template <typename T, int THREADS, int MAXV>
__global__ void __launch_bounds__(THREADS)
gated_norm_add_kernel(float* __restrict__ x, T* __restrict__ cast_out, const float* __restrict__ y, int n_sum,
                      const float* __restrict__ gate, int64_t gate_stride, const float* __restrict__ w, float eps, int normalize, int d, KeepRows keep,
                      const float* __restrict__ next_w, float next_eps) {
    __shared__ float red[THREADS / kWave];
    const int t = blockIdx.x;
    float* xr = x + static_cast<int64_t>(t) * d;
    if (keep.state != nullptr && t < *keep.n_real) {
        const int s = keep.tok_seq[t], p = keep.positions[t];
        const int slot = keep.state_slots[s];
        if (p >= keep.context_lens[s] - keep.ring && slot >= 0 && slot < keep.n_slots) {
            float* dst = keep.state + (static_cast<int64_t>(slot) * keep.ring + p % keep.ring) * d;
            for (int i = threadIdx.x; i < d; i += THREADS) dst[i] = xr[i];
        }
    }
    const float* yr = y + static_cast<int64_t>(t) * n_sum * d;
    const float* gr = gate != nullptr ? gate + static_cast<int64_t>(t) * gate_stride : nullptr;
    const bool held = d <= THREADS * MAXV;
    float sv[MAXV];
    float ss = 0.0f;
    auto value = [&](int i) {
        float s = yr[i];
        for (int k = 1; k < n_sum; ++k) s += yr[static_cast<int64_t>(k) * d + i];
        if (gr != nullptr) s *= sigmoidf(gr[i]);
        return s;
    };
    if (held) {
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int i = threadIdx.x + j * THREADS;
            sv[j] = i < d ? value(i) : 0.0f;
            ss += sv[j] * sv[j];
        }
    } else {
        for (int i = threadIdx.x; i < d; i += THREADS) {
            const float s = value(i);
            ss += s * s;
        }
    }
    const float scale = normalize ? 1.0f / sqrtf(rms_block_sum<THREADS>(ss, red) / static_cast<float>(d) + eps) : 1.0f;
    T* co = cast_out != nullptr ? cast_out + static_cast<int64_t>(t) * d : nullptr;
    const bool norm_next = next_w != nullptr && co != nullptr;  // what is written for the next product is the next norm of the new row
    float ss_new = 0.0f;
    auto finish = [&](int i, float s) {
        float v = s * scale;
        if (w != nullptr) v *= w[i];
        v += xr[i];
        xr[i] = v;
        if (norm_next) ss_new += v * v;
        else if (co != nullptr) co[i] = from_float<T>(v);
        return v;
    };
    if (held) {
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int i = threadIdx.x + j * THREADS;
            if (i < d) sv[j] = finish(i, sv[j]);
        }
    } else {
        for (int i = threadIdx.x; i < d; i += THREADS) finish(i, value(i));
    }
    if (norm_next) {
        const float next_scale = 1.0f / sqrtf(rms_block_sum<THREADS>(ss_new, red) / static_cast<float>(d) + next_eps);
        if (held) {
#pragma unroll
            for (int j = 0; j < MAXV; ++j) {
                const int i = threadIdx.x + j * THREADS;
                if (i < d) co[i] = from_float<T>(sv[j] * next_scale * next_w[i]);
            }
        } else {
            for (int i = threadIdx.x; i < d; i += THREADS) co[i] = from_float<T>(xr[i] * next_scale * next_w[i]);  // (each thread reads what it wrote)
        }
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_rmsnorm(void* out, int out_dtype, const float* x, const float* w, const int* rows, int n, int d, float eps,
                             hipStream_t stream) {
    LIYAB_REQUIRE(out && x, "rmsnorm: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0, "rmsnorm: bad sizes n=%d d=%d", n, d);
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "rmsnorm: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    if (out_dtype == kF32)
        rmsnorm_kernel<float, 256><<<n, 256, 0, stream>>>(static_cast<float*>(out), x, w, rows, d, eps);
    else
        rmsnorm_kernel<bf16_t, 256><<<n, 256, 0, stream>>>(static_cast<bf16_t*>(out), x, w, rows, d, eps);
    return check_launch("rmsnorm");
}

extern "C" int liyab_gated_norm_add(float* x, void* cast_out, int cast_dtype, const float* y, int n_sum, const float* gate,
                                    int64_t gate_stride, const float* w, float eps, int normalize, int n, int d, float* state, int ring, int n_slots,
                                    const int* tok_seq, const int* positions, const int* context_lens, const int* state_slots,
                                    const int* n_real, const float* next_w, float next_eps, hipStream_t stream) {
    LIYAB_REQUIRE(x && y, "gated_norm_add: null pointer");
    LIYAB_REQUIRE(next_w == nullptr || cast_out != nullptr, "gated_norm_add: the next norm's rows need a place");
    LIYAB_REQUIRE(n >= 0 && d > 0 && n_sum >= 1, "gated_norm_add: bad sizes n=%d d=%d n_sum=%d", n, d, n_sum);
    LIYAB_REQUIRE(cast_dtype == kF32 || cast_dtype == kBF16, "gated_norm_add: unknown dtype %d", cast_dtype);
    LIYAB_REQUIRE(gate == nullptr || gate_stride >= d, "gated_norm_add: the gate's row stride is shorter than a row");
    LIYAB_REQUIRE(state == nullptr || (ring > 0 && n_slots > 0 && tok_seq && positions && context_lens && state_slots && n_real),
                  "gated_norm_add: rows are kept only with a ring, slots and the step's tables");
    if (n == 0) return 0;
    const KeepRows keep{state, ring, n_slots, tok_seq, positions, context_lens, state_slots, n_real};
    if (cast_dtype == kF32)
        gated_norm_add_kernel<float, 256, 8><<<n, 256, 0, stream>>>(x, static_cast<float*>(cast_out), y, n_sum, gate, gate_stride, w, eps, normalize, d, keep, next_w, next_eps);
    else
        gated_norm_add_kernel<bf16_t, 256, 8><<<n, 256, 0, stream>>>(x, static_cast<bf16_t*>(cast_out), y, n_sum, gate, gate_stride, w, eps, normalize, d, keep, next_w, next_eps);
    return check_launch("gated_norm_add");
}
