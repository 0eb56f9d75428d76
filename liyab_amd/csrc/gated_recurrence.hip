// A linear recurrence a channel with real gates: S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t, with
// a = exp(-rate r softplus(lam)), r = s(zr + br), i = s(zi + bi) (s: the logistic function), zr and zi the products of u with a
// square matrix a part of the channels (`blocks` equal parts).
//
// liyab_lru_conv: u[t, c] = bias[c] + sum_j w[c, j] * x[t - taps + 1 + j, c] over a request's own rows in time (the last column
//   of w is the current row's; earlier rows from the step, or from the slot's ring where position p lies at place p % (taps - 1);
//   zeros before position 0). With `split`, u is also written as two bfloat16 numbers, u = hi + lo, part by part as [hi | lo]:
//   the gates' products then run on the matrix cores with the matrices twice side by side, [W W] [hi; lo] = W u to 16 bits of u,
//   where rounding u to one bfloat16 would move a decay that the recurrence multiplies by itself hundreds of times.
// liyab_lru_coeffs: decay and gated input of every token and channel from the gates' sums z (a part's [zr | zi] side by side), for
//   steps whose recurrence runs in stretches (below); 1 - a^2 is taken as -expm1(2 log a), which keeps its digits where a is near one.
// liyab_lru_scan: the walk. out[t] = out_scale * S_t * gelu_tanh(y_t) in the output type; the slot's S is read (zero at position 0,
//   whatever the slot holds) and left; the last taps - 1 rows of x take their places in the slot's ring (after the convolution,
//   which ran earlier on the stream, has read it). Two forms: a wave of 64 channels a request walks the request's rows in order
//   and takes decay and input from z as it goes (steps of few rows a request); or sixteen waves a workgroup, each a stretch of the
//   request's rows: every wave first walks its stretch from zero for the stretch's end and the product of its decays, the ends are
//   strung together through LDS, and every wave walks again from its true start (decay and input then come from liyab_lru_coeffs'
//   arrays). The recurrence is the same in the same 32-bit arithmetic, summed in another order. Rows behind the requests' own are
//   not touched. State, decays and sums are 32-bit.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int LS_WAVES = 16;

__device__ __forceinline__ float lru_logistic(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float lru_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float lru_gelu(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
// decay a and gated input b of one token and channel
__device__ __forceinline__ void lru_pair(float zr, float zi, float u, float cr, float ci, float sp, float rate, float& a, float& b) {
    const float la = -rate * lru_logistic(zr + cr) * sp;
    a = expf(la);
    b = sqrtf(-expm1f(2.0f * la)) * lru_logistic(zi + ci) * u;
}

__global__ void __launch_bounds__(256)
lru_conv_kernel(float* __restrict__ out, bf16_t* __restrict__ split, const float* __restrict__ in, int64_t ldi, const float* __restrict__ w,
                const float* __restrict__ bias, int taps, const float* __restrict__ state, int64_t state_stride, int n_slots,
                const int* __restrict__ tok_seq, const int* __restrict__ positions, const int* __restrict__ seq_starts,
                const int* __restrict__ state_slots, int C, int per) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int s = tok_seq[t], p = positions[t];
    const int begin = seq_starts[s];
    const int slot = state_slots[s];
    const bool slot_ok = slot >= 0 && slot < n_slots;
    const float* ring = state + static_cast<int64_t>(slot_ok ? slot : 0) * state_stride;
    float acc = bias != nullptr ? bias[c] : 0.0f;
    for (int jt = 0; jt < taps; ++jt) {
        const int back = taps - 1 - jt;  // rows before this one
        const int sp = p - back;
        if (sp < 0) continue;
        float x;
        if (t - back >= begin) x = in[static_cast<int64_t>(t - back) * ldi + c];
        else x = slot_ok ? ring[static_cast<int64_t>(sp % (taps - 1)) * C + c] : 0.0f;
        acc = fmaf(w[static_cast<int64_t>(c) * taps + jt], x, acc);
    }
    out[static_cast<int64_t>(t) * C + c] = acc;
    if (split != nullptr) {
        const bf16_t hi = float_to_bf16(acc);
        const bf16_t lo = float_to_bf16(acc - bf16_to_float(hi));
        bf16_t* dst = split + static_cast<int64_t>(t) * 2 * C + static_cast<int64_t>(c / per) * 2 * per + c % per;
        dst[0] = hi;
        dst[per] = lo;
    }
}

__global__ void __launch_bounds__(256)
lru_coeffs_kernel(float* __restrict__ decay, float* __restrict__ gated, const float* __restrict__ z, int64_t ldz, const float* __restrict__ u,
                  const float* __restrict__ br, const float* __restrict__ bi, const float* __restrict__ lam, float rate, int C, int per) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const float* zt = z + static_cast<int64_t>(t) * ldz + static_cast<int64_t>(c / per) * 2 * per + c % per;
    float a, b;
    lru_pair(zt[0], zt[per], u[static_cast<int64_t>(t) * C + c], br[c], bi[c], lru_softplus(lam[c]), rate, a, b);
    decay[static_cast<int64_t>(t) * C + c] = a;
    gated[static_cast<int64_t>(t) * C + c] = b;
}

struct LruScan {
    const float* z;  // the gates' sums [rows, ldz] (one wave a request), or null with decay and gated given (stretches)
    int64_t ldz;
    const float* u;
    const float* decay;
    const float* gated;
    const float *br, *bi, *lam;
    float rate, out_scale;
    const float* y;
    int64_t ldy;
    float* state;
    int64_t state_stride;
    int n_slots;
    const float* x;  // the convolution's input rows, of which the last taps - 1 are kept
    int64_t ldx;
    int taps;
    const int *seq_starts, *positions, *state_slots;
    int C, per;
};

// the last taps - 1 rows of the request's x (channel c) to their places in the ring behind S
__device__ __forceinline__ void lru_keep(const LruScan& p, float* slot_base, int begin, int end, int c) {
    const int places = p.taps - 1;
    for (int t = max(begin, end - places); t < end; ++t)
        slot_base[p.C + static_cast<int64_t>(p.positions[t] % places) * p.C + c] = p.x[static_cast<int64_t>(t) * p.ldx + c];
}

template <typename T>
__global__ void __launch_bounds__(64)
lru_scan_wave_kernel(T* __restrict__ out, LruScan p) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= p.C) return;
    const int begin = p.seq_starts[s], end = p.seq_starts[s + 1];
    if (end <= begin) return;
    const int slot = p.state_slots[s];
    const bool slot_ok = slot >= 0 && slot < p.n_slots;
    float* base = p.state + static_cast<int64_t>(slot_ok ? slot : 0) * p.state_stride;
    float S = (slot_ok && p.positions[begin] > 0) ? base[c] : 0.0f;
    const float cr = p.br[c], ci = p.bi[c], sp = lru_softplus(p.lam[c]);
    const int64_t zoff = static_cast<int64_t>(c / p.per) * 2 * p.per + c % p.per;
    int t = begin;
    // four tokens' operands are asked for before the first of them is used: the walk itself is one multiply-add a token
    for (; t + 4 <= end; t += 4) {
        float zr[4], zi[4], uu[4], g[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float* zt = p.z + static_cast<int64_t>(t + j) * p.ldz + zoff;
            zr[j] = zt[0];
            zi[j] = zt[p.per];
            uu[j] = p.u[static_cast<int64_t>(t + j) * p.C + c];
            g[j] = p.y[static_cast<int64_t>(t + j) * p.ldy + c];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a, b;
            lru_pair(zr[j], zi[j], uu[j], cr, ci, sp, p.rate, a, b);
            S = fmaf(a, S, b);
            out[static_cast<int64_t>(t + j) * p.C + c] = from_float<T>(p.out_scale * S * lru_gelu(g[j]));
        }
    }
    for (; t < end; ++t) {
        const float* zt = p.z + static_cast<int64_t>(t) * p.ldz + zoff;
        float a, b;
        lru_pair(zt[0], zt[p.per], p.u[static_cast<int64_t>(t) * p.C + c], cr, ci, sp, p.rate, a, b);
        S = fmaf(a, S, b);
        out[static_cast<int64_t>(t) * p.C + c] = from_float<T>(p.out_scale * S * lru_gelu(p.y[static_cast<int64_t>(t) * p.ldy + c]));
    }
    if (slot_ok) {
        base[c] = S;
        if (p.taps > 1) lru_keep(p, base, begin, end, c);
    }
}

template <typename T>
__global__ void __launch_bounds__(64 * LS_WAVES)
lru_scan_stretch_kernel(T* __restrict__ out, LruScan p) {
    __shared__ float prod[LS_WAVES][64], tail[LS_WAVES][64];
    const int s = blockIdx.y;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int c = blockIdx.x * 64 + lane;
    const bool c_ok = c < p.C;
    const int cc = c_ok ? c : p.C - 1;  // a lane past the channels walks the last one along; nothing of it is stored
    const int begin = p.seq_starts[s], end = p.seq_starts[s + 1];
    const int len = max(end - begin, 0);
    const int chunk = (len + LS_WAVES - 1) / LS_WAVES;
    const int t0 = min(end, begin + wave * chunk), t1 = min(end, t0 + chunk);
    const int slot = p.state_slots[s];
    const bool slot_ok = slot >= 0 && slot < p.n_slots;
    float* base = p.state + static_cast<int64_t>(slot_ok ? slot : 0) * p.state_stride;
    // the stretch from zero: its end and the product of its decays
    float P = 1.0f, Z = 0.0f;
    int t = t0;
    for (; t + 4 <= t1; t += 4) {
        float a[4], b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = p.decay[static_cast<int64_t>(t + j) * p.C + cc];
            b[j] = p.gated[static_cast<int64_t>(t + j) * p.C + cc];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            Z = fmaf(a[j], Z, b[j]);
            P *= a[j];
        }
    }
    for (; t < t1; ++t) {
        const float a = p.decay[static_cast<int64_t>(t) * p.C + cc];
        Z = fmaf(a, Z, p.gated[static_cast<int64_t>(t) * p.C + cc]);
        P *= a;
    }
    prod[wave][lane] = P;
    tail[wave][lane] = Z;
    __syncthreads();
    // the state this stretch starts from: the request's own, then the stretches before it in their order
    float S = (slot_ok && len > 0 && p.positions[begin] > 0) ? base[cc] : 0.0f;
    for (int w = 0; w < wave; ++w) S = fmaf(prod[w][lane], S, tail[w][lane]);
    t = t0;
    for (; t + 4 <= t1; t += 4) {
        float a[4], b[4], g[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = p.decay[static_cast<int64_t>(t + j) * p.C + cc];
            b[j] = p.gated[static_cast<int64_t>(t + j) * p.C + cc];
            g[j] = p.y[static_cast<int64_t>(t + j) * p.ldy + cc];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            S = fmaf(a[j], S, b[j]);
            if (c_ok) out[static_cast<int64_t>(t + j) * p.C + c] = from_float<T>(p.out_scale * S * lru_gelu(g[j]));
        }
    }
    for (; t < t1; ++t) {
        S = fmaf(p.decay[static_cast<int64_t>(t) * p.C + cc], S, p.gated[static_cast<int64_t>(t) * p.C + cc]);
        if (c_ok) out[static_cast<int64_t>(t) * p.C + c] = from_float<T>(p.out_scale * S * lru_gelu(p.y[static_cast<int64_t>(t) * p.ldy + cc]));
    }
    // the last wave's end is the request's (a wave without rows carries the state through: its product is one, its end zero)
    if (wave == LS_WAVES - 1 && c_ok && slot_ok && len > 0) {
        base[c] = S;
        if (p.taps > 1) lru_keep(p, base, begin, end, c);
    }
}

}  // namespace liyab

using namespace liyab;

// out: float [n, C]; split: bfloat16 [n, 2 C] or null; in: float rows [n, ldi]; w: float [C, taps]; bias: float [C] or null; state: the
// slots' ring at its first float (the caller adds the ring's offset), state_stride floats between slots.
extern "C" int liyab_lru_conv(float* out, void* split, const float* in, int64_t ldi, const float* w, const float* bias, int taps, const float* state,
                              int64_t state_stride, int n_slots, const int* tok_seq, const int* positions, const int* seq_starts,
                              const int* state_slots, int n, int C, int blocks, hipStream_t stream) {
    LIYAB_REQUIRE(out && in && w && tok_seq && positions && seq_starts && state_slots, "lru_conv: null pointer");
    LIYAB_REQUIRE(n >= 0 && n <= 65535 && C > 0 && taps >= 1 && ldi >= C && blocks >= 1 && C % blocks == 0, "lru_conv: bad sizes");
    LIYAB_REQUIRE(taps == 1 || (state != nullptr && n_slots > 0 && state_stride >= static_cast<int64_t>(taps - 1) * C),
                  "lru_conv: %d taps need the last %d rows of a request in its slot", taps, taps - 1);
    if (n == 0) return 0;
    dim3 grid((C + 255) / 256, n);
    lru_conv_kernel<<<grid, 256, 0, stream>>>(out, static_cast<bf16_t*>(split), in, ldi, w, bias, taps, state, state_stride, taps > 1 ? n_slots : 0, tok_seq,
                                              positions, seq_starts, state_slots, C, C / blocks);
    return check_launch("lru_conv");
}

// decay, gated: float [n, C]; z: float rows [n, ldz], a part's sums as [zr | zi]; u: float [n, C]; br, bi, lam: float [C].
extern "C" int liyab_lru_coeffs(float* decay, float* gated, const float* z, int64_t ldz, const float* u, const float* br, const float* bi,
                                const float* lam, float rate, int n, int C, int blocks, hipStream_t stream) {
    LIYAB_REQUIRE(decay && gated && z && u && br && bi && lam, "lru_coeffs: null pointer");
    LIYAB_REQUIRE(n >= 0 && n <= 65535 && C > 0 && blocks >= 1 && C % blocks == 0 && ldz >= 2 * static_cast<int64_t>(C), "lru_coeffs: bad sizes");
    if (n == 0) return 0;
    dim3 grid((C + 255) / 256, n);
    lru_coeffs_kernel<<<grid, 256, 0, stream>>>(decay, gated, z, ldz, u, br, bi, lam, rate, C, C / blocks);
    return check_launch("lru_coeffs");
}

// out [rows, C] in out_dtype. stretches = 0: z (float rows [rows, ldz]) and u (float [rows, C]) are read, decay and gated are not;
// stretches = 1: decay and gated (float [rows, C], from liyab_lru_coeffs) are read. y: float rows [rows, ldy]; state: float
// [n_slots, state_stride], a request's S in the first C floats of its slot, the ring of taps - 1 rows of x (float rows [rows, ldx])
// behind it.
extern "C" int liyab_lru_scan(void* out, int out_dtype, const float* z, int64_t ldz, const float* u, const float* decay, const float* gated,
                              const float* br, const float* bi, const float* lam, float rate, float out_scale, const float* y, int64_t ldy,
                              float* state, int64_t state_stride, int n_slots, const float* x, int64_t ldx, int taps, const int* seq_starts,
                              const int* positions, const int* state_slots, int n_seqs, int C, int blocks, int stretches, hipStream_t stream) {
    LIYAB_REQUIRE(out && y && state && seq_starts && positions && state_slots && br && bi && lam, "lru_scan: null pointer");
    LIYAB_REQUIRE(stretches ? (decay && gated) : (z && u), "lru_scan: the walk's operands are missing");
    LIYAB_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && C > 0 && blocks >= 1 && C % blocks == 0 && ldy >= C && n_slots > 0 && taps >= 1, "lru_scan: bad sizes");
    LIYAB_REQUIRE(stretches || ldz >= 2 * static_cast<int64_t>(C), "lru_scan: the gates' rows are shorter than two a channel");
    LIYAB_REQUIRE(state_stride >= static_cast<int64_t>(taps) * C && (taps == 1 || (x != nullptr && ldx >= C)), "lru_scan: the slot does not hold the state and %d rows", taps - 1);
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "lru_scan: unknown dtype %d", out_dtype);
    if (n_seqs == 0) return 0;
    const LruScan p{z, ldz, u, decay, gated, br, bi, lam, rate, out_scale, y, ldy, state, state_stride, n_slots, x, ldx, taps, seq_starts, positions, state_slots, C, C / blocks};
    const dim3 grid((C + 63) / 64, n_seqs);
    if (stretches) {
        if (out_dtype == kF32) lru_scan_stretch_kernel<float><<<grid, 64 * LS_WAVES, 0, stream>>>(static_cast<float*>(out), p);
        else lru_scan_stretch_kernel<bf16_t><<<grid, 64 * LS_WAVES, 0, stream>>>(static_cast<bf16_t*>(out), p);
    } else {
        if (out_dtype == kF32) lru_scan_wave_kernel<float><<<grid, 64, 0, stream>>>(static_cast<float*>(out), p);
        else lru_scan_wave_kernel<bf16_t><<<grid, 64, 0, stream>>>(static_cast<bf16_t*>(out), p);
    }
    return check_launch("lru_scan");
}
