// A linear recurrence a channel with real gates: S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t.
//
// liyab_lru_gates: from the recurrence's input u (32-bit rows, `width` channels in `blocks` equal parts) the decay and the
//   gated input of every token and channel. In part b: r = s(Wr[b] u_b + br), i = s(Wi[b] u_b + bi) (s: the logistic
//   function; Wr[b], Wi[b] square, stored [part][in][out], so that threads side by side read outputs side by side);
//   log a = -rate r softplus(lam); decay = exp(log a); input = sqrt(1 - a^2) i u, with 1 - a^2 taken as -expm1(2 log a), which
//   keeps its digits where a is near one. Weights bfloat16 or 32-bit; u, sums and everything behind them 32-bit.
//   A workgroup takes 16 tokens x 64 outputs of one part; a thread 4 tokens of one output, both gates; u goes through LDS
//   64 inputs at a time.
// liyab_lru_scan: a thread a (request, channel) walks the request's rows of the step in order from the slot's state
//   (zero at position 0, whatever the slot holds), writes S_t * gelu_tanh(y_t) in the output type and leaves the last S in
//   the slot. Rows behind the requests' own are not touched. State and sums 32-bit.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int LG_TOKENS = 16, LG_OUT = 64, LG_K = 64;

__device__ __forceinline__ float lru_logistic(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float lru_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float lru_gelu(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename W>
__global__ void __launch_bounds__(256)
lru_gates_kernel(float* __restrict__ decay, float* __restrict__ input, const float* __restrict__ u, int64_t ldu, const W* __restrict__ wr,
                 const W* __restrict__ wi, const float* __restrict__ br, const float* __restrict__ bi, const float* __restrict__ lam,
                 float rate, int n, int width, int per) {
    __shared__ float us[LG_TOKENS][LG_K + 1];
    const int t0 = blockIdx.x * LG_TOKENS, b = blockIdx.y, o0 = blockIdx.z * LG_OUT;
    const int tid = threadIdx.x, ol = tid % LG_OUT, tg = tid / LG_OUT;
    const int o = o0 + ol;
    const bool o_ok = o < per;
    const int oc = o_ok ? o : per - 1;  // an output past the part's end reads the last one's weights; never stored
    const W* wrb = wr + static_cast<int64_t>(b) * per * per + oc;
    const W* wib = wi + static_cast<int64_t>(b) * per * per + oc;
    float ar[4] = {0.0f, 0.0f, 0.0f, 0.0f}, ai[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int k0 = 0; k0 < per; k0 += LG_K) {
        __syncthreads();
        for (int e = tid; e < LG_TOKENS * LG_K; e += 256) {
            const int tt = e / LG_K, k = e % LG_K;
            const int t = t0 + tt;
            us[tt][k] = (t < n && k0 + k < per) ? u[static_cast<int64_t>(t) * ldu + b * per + k0 + k] : 0.0f;
        }
        __syncthreads();
        const int kn = min(LG_K, per - k0);
        for (int k = 0; k < kn; ++k) {
            const float vr = to_float<W>(wrb[static_cast<int64_t>(k0 + k) * per]);
            const float vi = to_float<W>(wib[static_cast<int64_t>(k0 + k) * per]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float x = us[tg * 4 + j][k];
                ar[j] = fmaf(vr, x, ar[j]);
                ai[j] = fmaf(vi, x, ai[j]);
            }
        }
    }
    if (!o_ok) return;
    const int c = b * per + o;
    const float sp = lru_softplus(lam[c]), cr = br[c], ci = bi[c];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int t = t0 + tg * 4 + j;
        if (t >= n) continue;
        const float r = lru_logistic(ar[j] + cr), g = lru_logistic(ai[j] + ci);
        const float la = -rate * r * sp;
        const float x = u[static_cast<int64_t>(t) * ldu + c];
        decay[static_cast<int64_t>(t) * width + c] = expf(la);
        input[static_cast<int64_t>(t) * width + c] = sqrtf(-expm1f(2.0f * la)) * g * x;
    }
}

template <typename T>
__global__ void __launch_bounds__(64)
lru_scan_kernel(T* __restrict__ out, const float* __restrict__ decay, const float* __restrict__ input, const float* __restrict__ y, int64_t ldy,
                float* __restrict__ state, int64_t state_stride, int n_slots, const int* __restrict__ seq_starts,
                const int* __restrict__ positions, const int* __restrict__ state_slots, int width) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= width) return;
    const int begin = seq_starts[s], end = seq_starts[s + 1];
    if (end <= begin) return;
    const int slot = state_slots[s];
    const bool slot_ok = slot >= 0 && slot < n_slots;
    float* st = state + static_cast<int64_t>(slot_ok ? slot : 0) * state_stride + c;
    float S = (slot_ok && positions[begin] > 0) ? *st : 0.0f;
    int t = begin;
    // four tokens' operands are asked for before the first of them is used: the walk itself is one multiply-add a token
    for (; t + 4 <= end; t += 4) {
        float a[4], b[4], g[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = decay[static_cast<int64_t>(t + j) * width + c];
            b[j] = input[static_cast<int64_t>(t + j) * width + c];
            g[j] = y[static_cast<int64_t>(t + j) * ldy + c];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            S = fmaf(a[j], S, b[j]);
            out[static_cast<int64_t>(t + j) * width + c] = from_float<T>(S * lru_gelu(g[j]));
        }
    }
    for (; t < end; ++t) {
        S = fmaf(decay[static_cast<int64_t>(t) * width + c], S, input[static_cast<int64_t>(t) * width + c]);
        out[static_cast<int64_t>(t) * width + c] = from_float<T>(S * lru_gelu(y[static_cast<int64_t>(t) * ldy + c]));
    }
    if (slot_ok) *st = S;
}

}  // namespace liyab

using namespace liyab;

// decay, input: float [n, width]; u: float rows [n, ldu]; wr, wi: [blocks, width / blocks (in), width / blocks (out)] in w_dtype;
// br, bi, lam: float [width].
extern "C" int liyab_lru_gates(float* decay, float* input, const float* u, int64_t ldu, const void* wr, const void* wi, int w_dtype, const float* br,
                               const float* bi, const float* lam, float rate, int n, int blocks, int width, hipStream_t stream) {
    LIYAB_REQUIRE(decay && input && u && wr && wi && br && bi && lam, "lru_gates: null pointer");
    LIYAB_REQUIRE(n >= 0 && blocks > 0 && blocks <= 65535 && width > 0 && width % blocks == 0 && ldu >= width, "lru_gates: bad sizes (%d channels in %d parts)", width, blocks);
    LIYAB_REQUIRE(w_dtype == kF32 || w_dtype == kBF16, "lru_gates: unknown dtype %d", w_dtype);
    if (n == 0) return 0;
    const int per = width / blocks;
    LIYAB_REQUIRE((per + LG_OUT - 1) / LG_OUT <= 65535, "lru_gates: parts of %d channels", per);
    const dim3 grid((n + LG_TOKENS - 1) / LG_TOKENS, blocks, (per + LG_OUT - 1) / LG_OUT);
    if (w_dtype == kF32)
        lru_gates_kernel<float><<<grid, 256, 0, stream>>>(decay, input, u, ldu, static_cast<const float*>(wr), static_cast<const float*>(wi), br, bi, lam, rate, n,
                                                          width, per);
    else
        lru_gates_kernel<bf16_t><<<grid, 256, 0, stream>>>(decay, input, u, ldu, static_cast<const bf16_t*>(wr), static_cast<const bf16_t*>(wi), br, bi, lam, rate,
                                                           n, width, per);
    return check_launch("lru_gates");
}

// out [rows, width] in out_dtype; decay, input: float [rows, width]; y: float rows [rows, ldy]; state: float [n_slots, state_stride],
// a request's S in the first `width` floats of its slot.
extern "C" int liyab_lru_scan(void* out, int out_dtype, const float* decay, const float* input, const float* y, int64_t ldy, float* state,
                              int64_t state_stride, int n_slots, const int* seq_starts, const int* positions, const int* state_slots, int n_seqs,
                              int width, hipStream_t stream) {
    LIYAB_REQUIRE(out && decay && input && y && state && seq_starts && positions && state_slots, "lru_scan: null pointer");
    LIYAB_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && width > 0 && ldy >= width && n_slots > 0 && state_stride >= width, "lru_scan: bad sizes");
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "lru_scan: unknown dtype %d", out_dtype);
    if (n_seqs == 0) return 0;
    const dim3 grid((width + 63) / 64, n_seqs);
    if (out_dtype == kF32)
        lru_scan_kernel<float><<<grid, 64, 0, stream>>>(static_cast<float*>(out), decay, input, y, ldy, state, state_stride, n_slots, seq_starts, positions,
                                                        state_slots, width);
    else
        lru_scan_kernel<bf16_t><<<grid, 64, 0, stream>>>(static_cast<bf16_t*>(out), decay, input, y, ldy, state, state_stride, n_slots, seq_starts, positions,
                                                         state_slots, width);
    return check_launch("lru_scan");
}
