// Norms without statistics, gated activations and the joining of two sublayers' results.
//
// liyab_dyt: the Dynamic Tanh norm, y = tanh(alpha * x) * w + b over rows of the 32-bit residual
// stream: no mean and no variance, one learned scalar alpha (read from device memory), a weight
// and a bias a channel. `rows`, when given, gathers (the final norm runs on the wanted rows only).
//
// liyab_glu_clamped: the inner rows of a gated feed-forward whose two halves are clamped before
// they meet: g = min(G, limit), u = clamp(U, -limit, limit), y = g * sigmoid(slope * g) * (u + shift),
// from one 32-bit product [G | U] a row.
//
// liyab_activate: tanh, silu, the logistic function or the squared positive part of 32-bit rows, rounded to the output type.
//
// liyab_gate_rows: x *= scale * sigmoid(g) in place, a gate on a mixer's rows from 32-bit logits (and a constant factor).
//
// liyab_mean_norm_add: x += weight * (a / rms(a) * wa + b / rms(b) * wb), the two results of
// sublayers that run side by side, each brought to unit root mean square over the row first.
//
// liyab_weighted_sum: out = wa * a + wb * b, two sublayers' results joined with constant weights.
//
// All arithmetic is 32-bit; a result is rounded once, to the output type.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int EW_THREADS = 256;

__device__ __forceinline__ float logistic(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ void __launch_bounds__(EW_THREADS)
dyt_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ b,
           const float* __restrict__ alpha, const int* __restrict__ rows, int d) {
    const int r = blockIdx.x;
    const int64_t src = rows != nullptr ? rows[r] : r;
    const float a = alpha[0];
    const float* xr = x + src * d;
    T* o = out + static_cast<int64_t>(r) * d;
    for (int i = threadIdx.x; i < d; i += EW_THREADS) {
        float v = tanhf(a * xr[i]);
        if (w != nullptr) v *= w[i];
        if (b != nullptr) v += b[i];
        o[i] = from_float<T>(v);
    }
}

template <typename T>
__global__ void __launch_bounds__(EW_THREADS)
glu_clamped_kernel(T* __restrict__ out, const float* __restrict__ gu, int64_t ld, int ff, float limit, float slope, float shift) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * EW_THREADS + threadIdx.x;
    if (i >= ff) return;
    const float* row = gu + static_cast<int64_t>(t) * ld;
    const float g = fminf(row[i], limit);
    const float u = fminf(fmaxf(row[ff + i], -limit), limit);
    out[static_cast<int64_t>(t) * ff + i] = from_float<T>(g * logistic(slope * g) * (u + shift));
}

template <typename T>
__global__ void __launch_bounds__(EW_THREADS)
activate_kernel(T* __restrict__ out, int64_t ldo, const float* __restrict__ in, int64_t ldi, int op, int d) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * EW_THREADS + threadIdx.x;
    if (i >= d) return;
    const float z = in[static_cast<int64_t>(t) * ldi + i];
    const float v = op == 0 ? tanhf(z) : op == 1 ? z * logistic(z) : op == 2 ? logistic(z) : (z > 0.0f ? z * z : 0.0f);
    out[static_cast<int64_t>(t) * ldo + i] = from_float<T>(v);
}

template <typename T>
__global__ void __launch_bounds__(EW_THREADS)
gate_rows_kernel(T* __restrict__ x, int64_t ldx, const float* __restrict__ gate, int64_t ldg, int d, float scale) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * EW_THREADS + threadIdx.x;
    if (i >= d) return;
    T* at = x + static_cast<int64_t>(t) * ldx + i;
    *at = from_float<T>(to_float<T>(*at) * logistic(gate[static_cast<int64_t>(t) * ldg + i]) * scale);
}

__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < EW_THREADS / kWave; ++i) total += red[i];
    return total;
}

__global__ void __launch_bounds__(EW_THREADS)
mean_norm_add_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ wa,
                     const float* __restrict__ wb, float eps, float weight, int d) {
    __shared__ float red[EW_THREADS / kWave];
    const int64_t row = static_cast<int64_t>(blockIdx.x) * d;
    float sa = 0.0f, sb = 0.0f;
    for (int i = threadIdx.x; i < d; i += EW_THREADS) {
        sa += a[row + i] * a[row + i];
        sb += b[row + i] * b[row + i];
    }
    const float ra = 1.0f / sqrtf(block_sum(sa, red) / static_cast<float>(d) + eps);
    const float rb = 1.0f / sqrtf(block_sum(sb, red) / static_cast<float>(d) + eps);
    for (int i = threadIdx.x; i < d; i += EW_THREADS)
        x[row + i] += weight * (a[row + i] * ra * wa[i] + b[row + i] * rb * wb[i]);
}

__global__ void __launch_bounds__(EW_THREADS)
weighted_sum_kernel(float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ b, float wa, float wb, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * EW_THREADS + threadIdx.x;
    if (i < n) out[i] = wa * a[i] + wb * b[i];
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_weighted_sum(float* out, const float* a, const float* b, float wa, float wb, int64_t n, hipStream_t stream) {
    LIYAB_REQUIRE(out && a && b, "weighted_sum: null pointer");
    LIYAB_REQUIRE(n >= 0 && n < (int64_t(1) << 38), "weighted_sum: bad size");
    if (n == 0) return 0;
    weighted_sum_kernel<<<static_cast<unsigned>((n + EW_THREADS - 1) / EW_THREADS), EW_THREADS, 0, stream>>>(out, a, b, wa, wb, n);
    return check_launch("weighted_sum");
}

extern "C" int liyab_dyt(void* out, int out_dtype, const float* x, const float* w, const float* b, const float* alpha, const int* rows,
                         int n, int d, hipStream_t stream) {
    LIYAB_REQUIRE(out && x && alpha, "dyt: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0, "dyt: bad sizes");
    if (n == 0) return 0;
    if (out_dtype == kF32) dyt_kernel<float><<<n, EW_THREADS, 0, stream>>>(static_cast<float*>(out), x, w, b, alpha, rows, d);
    else if (out_dtype == kBF16) dyt_kernel<bf16_t><<<n, EW_THREADS, 0, stream>>>(static_cast<bf16_t*>(out), x, w, b, alpha, rows, d);
    else return fail(1, "dyt: unknown dtype %d", out_dtype);
    return check_launch("dyt");
}

extern "C" int liyab_glu_clamped(void* out, int out_dtype, const float* gu, int64_t ld, int n, int ff, float limit, float slope, float shift,
                                 hipStream_t stream) {
    LIYAB_REQUIRE(out && gu, "glu_clamped: null pointer");
    LIYAB_REQUIRE(n >= 0 && n <= 65535 && ff > 0 && ld >= 2 * static_cast<int64_t>(ff), "glu_clamped: bad sizes");
    LIYAB_REQUIRE(limit > 0.0f, "glu_clamped: the limit must be positive");
    if (n == 0) return 0;
    dim3 grid((ff + EW_THREADS - 1) / EW_THREADS, n);
    if (out_dtype == kF32) glu_clamped_kernel<float><<<grid, EW_THREADS, 0, stream>>>(static_cast<float*>(out), gu, ld, ff, limit, slope, shift);
    else if (out_dtype == kBF16) glu_clamped_kernel<bf16_t><<<grid, EW_THREADS, 0, stream>>>(static_cast<bf16_t*>(out), gu, ld, ff, limit, slope, shift);
    else return fail(1, "glu_clamped: unknown dtype %d", out_dtype);
    return check_launch("glu_clamped");
}

extern "C" int liyab_activate(void* out, int out_dtype, int64_t ldo, const float* in, int64_t ldi, int op, int n, int d, hipStream_t stream) {
    LIYAB_REQUIRE(out && in, "activate: null pointer");
    LIYAB_REQUIRE(n >= 0 && n <= 65535 && d > 0 && ldo >= d && ldi >= d, "activate: bad sizes");
    LIYAB_REQUIRE(op >= 0 && op <= 3, "activate: unknown function %d", op);
    if (n == 0) return 0;
    dim3 grid((d + EW_THREADS - 1) / EW_THREADS, n);
    if (out_dtype == kF32) activate_kernel<float><<<grid, EW_THREADS, 0, stream>>>(static_cast<float*>(out), ldo, in, ldi, op, d);
    else if (out_dtype == kBF16) activate_kernel<bf16_t><<<grid, EW_THREADS, 0, stream>>>(static_cast<bf16_t*>(out), ldo, in, ldi, op, d);
    else return fail(1, "activate: unknown dtype %d", out_dtype);
    return check_launch("activate");
}

// x[t, i] *= scale * sigmoid(gate[t, i]) in place; x rows in float32 or bfloat16, gate float32 logits.
extern "C" int liyab_gate_rows(void* x, int dtype, int64_t ldx, const float* gate, int64_t ldg, int n, int d, float scale, hipStream_t stream) {
    LIYAB_REQUIRE(x && gate, "gate_rows: null pointer");
    LIYAB_REQUIRE(n >= 0 && n <= 65535 && d > 0 && ldx >= d && ldg >= d, "gate_rows: bad sizes");
    if (n == 0) return 0;
    dim3 grid((d + EW_THREADS - 1) / EW_THREADS, n);
    if (dtype == kF32) gate_rows_kernel<float><<<grid, EW_THREADS, 0, stream>>>(static_cast<float*>(x), ldx, gate, ldg, d, scale);
    else if (dtype == kBF16) gate_rows_kernel<bf16_t><<<grid, EW_THREADS, 0, stream>>>(static_cast<bf16_t*>(x), ldx, gate, ldg, d, scale);
    else return fail(1, "gate_rows: unknown dtype %d", dtype);
    return check_launch("gate_rows");
}

extern "C" int liyab_mean_norm_add(float* x, const float* a, const float* b, const float* wa, const float* wb, float eps, float weight, int n,
                                   int d, hipStream_t stream) {
    LIYAB_REQUIRE(x && a && b && wa && wb, "mean_norm_add: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0, "mean_norm_add: bad sizes");
    if (n == 0) return 0;
    mean_norm_add_kernel<<<n, EW_THREADS, 0, stream>>>(x, a, b, wa, wb, eps, weight, d);
    return check_launch("mean_norm_add");
}
