// A recurrence that decays a head's matrix of state and takes out of it what the token's key already holds there, before the
// token's own outer product is added (a delta rule with a decay and a removal rate a channel):
//   u = k / sqrt(sum(k^2) + key_eps),   w = exp(-decay_scale * sigmoid(wraw + w0)),   a = sigmoid(araw + a_bias)
//   S <- diag(w) S - (a * u)(u^T S) + k v^T         (both terms read the old S; S is [key channel, value channel])
//   o = S^T r
// The map S -> diag(w) S - (a * u)(u^T S) acts on every column of S on its own, so columns never exchange anything.
//
// liyab_delta_prepare: (w, a * u, u) of every token, head and key channel, float32 [n, 3, H * D]: a wave a (token, head).
// liyab_delta_scan: a wave a (request, head, block of 16 columns) walks the request's rows of the step in order. Four lanes
//   side by side share a column, each with a quarter of its rows in registers, so the two sums over the rows of a column
//   (u^T S and S^T r) are sums over a quad of lanes, which come through the lanes' own data path; nothing goes through
//   LDS and no wave waits for another. A token's operands are fetched while the token before it is computed. The state is
//   32-bit in the request's slot and in registers; it is zero at position 0 whatever the slot holds.
// liyab_head_norm_gate: out = o / sqrt(mean(o^2 over the head) + eps) * weight * sigmoid(gate), rounded once.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kDeltaCols = 16;    // columns of S a wave
constexpr int kDeltaSplit = 4;    // lanes that share a column's rows
constexpr int kDeltaWaves = 4;    // waves a workgroup, each with work of its own

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

__global__ void __launch_bounds__(256)
delta_prepare_kernel(float* __restrict__ prep, const float* __restrict__ k, const float* __restrict__ wraw, const float* __restrict__ araw,
                     int64_t ld, int64_t ldw, const float* __restrict__ w0, const float* __restrict__ a_bias, float decay_scale, float key_eps,
                     int n, int H, int D) {
    const int item = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (item >= n * H) return;
    const int t = item / H, h = item % H;
    const float* kr = k + static_cast<int64_t>(t) * ld + h * D;
    float ss = 0.0f;
    for (int i = lane; i < D; i += kWave) ss += kr[i] * kr[i];
    const float inv = 1.0f / sqrtf(wave_sum(ss) + key_eps);
    const int64_t HD = static_cast<int64_t>(H) * D;
    float* o = prep + static_cast<int64_t>(t) * 3 * HD + h * D;
    for (int i = lane; i < D; i += kWave) {
        const float u = kr[i] * inv;
        const float w = expf(-decay_scale * sigmoid_f(wraw[static_cast<int64_t>(t) * ldw + h * D + i] + w0[h * D + i]));
        const float a = sigmoid_f(araw[static_cast<int64_t>(t) * ld + h * D + i] + a_bias[h * D + i]);
        o[i] = w;
        o[HD + i] = a * u;
        o[2 * HD + i] = u;
    }
}

struct DeltaArgs {
    float* out;               // [n, H * D] float32
    const float *r, *k, *v;   // rows of ld floats, a head's D values at h * D
    int64_t ld;
    const float* prep;        // [n, 3, H * D]
    float* state;             // the heads' matrices [H, D, D] of slot 0; a slot is state_stride floats further
    int64_t state_stride;
    int n_slots;
    const int* seq_starts;
    const int* positions;
    const int* state_slots;
    int n_seqs, H, D;
};

// REG: rows a lane holds (D <= 4 * REG); a lane's rows are i0 .. i0 + REG - 1, i0 = (lane % 4) * REG
template <int REG>
struct DeltaOperands {
    float w[REG], au[REG], u[REG], k[REG], r[REG];
    float v;
};

template <int REG>
__device__ __forceinline__ void delta_fetch(DeltaOperands<REG>& op, const DeltaArgs& a, int t, int h, int i0, int j) {
    const int D = a.D;
    const int64_t HD = static_cast<int64_t>(a.H) * D;
    const float* p = a.prep + static_cast<int64_t>(t) * 3 * HD + h * D;
    const float* kr = a.k + static_cast<int64_t>(t) * a.ld + h * D;
    const float* rr = a.r + static_cast<int64_t>(t) * a.ld + h * D;
#pragma unroll
    for (int ii = 0; ii < REG; ++ii) {
        const int i = min(i0 + ii, D - 1);  // (rows past the head's last read its last and are masked where they are used)
        op.w[ii] = p[i];
        op.au[ii] = p[HD + i];
        op.u[ii] = p[2 * HD + i];
        op.k[ii] = kr[i];
        op.r[ii] = rr[i];
    }
    op.v = a.v[static_cast<int64_t>(t) * a.ld + h * D + min(j, D - 1)];
}

template <int REG, bool AHEAD>
__global__ void __launch_bounds__(kDeltaWaves * kWave)
delta_scan_kernel(DeltaArgs a) {
    const int lane = threadIdx.x % kWave;
    const int n_cb = (a.D + kDeltaCols - 1) / kDeltaCols;
    const int item = blockIdx.x * kDeltaWaves + threadIdx.x / kWave;
    if (item >= a.n_seqs * a.H * n_cb) return;
    const int cb = item % n_cb, h = (item / n_cb) % a.H, s = item / (n_cb * a.H);
    const int begin = a.seq_starts[s], end = a.seq_starts[s + 1];
    if (begin >= end) return;
    const int D = a.D;
    const int rb = lane % kDeltaSplit, j = cb * kDeltaCols + lane / kDeltaSplit;
    const int i0 = rb * REG;
    const int slot = a.state_slots[s];
    const bool slot_ok = slot >= 0 && slot < a.n_slots;
    const bool fresh = a.positions[begin] == 0;
    float* Sg = a.state + static_cast<int64_t>(slot_ok ? slot : 0) * a.state_stride + static_cast<int64_t>(h) * D * D;
    float S[REG];
    bool mine[REG];
#pragma unroll
    for (int ii = 0; ii < REG; ++ii) {
        mine[ii] = i0 + ii < D && j < D;
        S[ii] = (mine[ii] && slot_ok && !fresh) ? Sg[static_cast<int64_t>(i0 + ii) * D + j] : 0.0f;
    }
    DeltaOperands<REG> cur, nxt;
    delta_fetch<REG>(cur, a, begin, h, i0, j);
    for (int t = begin; t < end; ++t) {
        if (AHEAD) delta_fetch<REG>(nxt, a, min(t + 1, end - 1), h, i0, j);
        float seen = 0.0f;
#pragma unroll
        for (int ii = 0; ii < REG; ++ii) seen += mine[ii] ? cur.u[ii] * S[ii] : 0.0f;
        seen = group_sum<kDeltaSplit>(seen);
        float o = 0.0f;
#pragma unroll
        for (int ii = 0; ii < REG; ++ii) {
            S[ii] = mine[ii] ? cur.w[ii] * S[ii] - cur.au[ii] * seen + cur.k[ii] * cur.v : 0.0f;
            o += cur.r[ii] * S[ii];
        }
        o = group_sum<kDeltaSplit>(o);
        if (rb == 0 && j < D) a.out[static_cast<int64_t>(t) * a.H * D + h * D + j] = o;
        if (AHEAD) cur = nxt;
        else if (t + 1 < end) delta_fetch<REG>(cur, a, t + 1, h, i0, j);
    }
    if (slot_ok) {
#pragma unroll
        for (int ii = 0; ii < REG; ++ii)
            if (mine[ii]) Sg[static_cast<int64_t>(i0 + ii) * D + j] = S[ii];
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ gate, int64_t ldg, const float* __restrict__ w,
                      float eps, int n, int H, int D) {
    const int item = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (item >= n * H) return;
    const int t = item / H, h = item % H;
    const float* row = o + (static_cast<int64_t>(t) * H + h) * D;
    float ss = 0.0f;
    for (int i = lane; i < D; i += kWave) ss += row[i] * row[i];
    const float scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + eps);
    for (int i = lane; i < D; i += kWave) {
        float v = row[i] * scale;
        if (w != nullptr) v *= w[h * D + i];
        if (gate != nullptr) v *= sigmoid_f(gate[static_cast<int64_t>(t) * ldg + h * D + i]);
        out[(static_cast<int64_t>(t) * H + h) * D + i] = from_float<T>(v);
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_delta_takes(int D) { return D >= 1 && D <= 256 ? 1 : 0; }

extern "C" int liyab_delta_prepare(float* prep, const float* k, const float* wraw, const float* araw, int64_t ld, int64_t ldw, const float* w0,
                                   const float* a_bias, float decay_scale, float key_eps, int n, int H, int D, hipStream_t stream) {
    LIYAB_REQUIRE(prep && k && wraw && araw && w0 && a_bias, "delta_prepare: null pointer");
    LIYAB_REQUIRE(n >= 0 && H > 0 && D > 0 && ld >= static_cast<int64_t>(H) * D && ldw >= static_cast<int64_t>(H) * D, "delta_prepare: bad sizes");
    if (n == 0) return 0;
    const int64_t items = static_cast<int64_t>(n) * H;
    delta_prepare_kernel<<<static_cast<unsigned>((items + 3) / 4), 256, 0, stream>>>(prep, k, wraw, araw, ld, ldw, w0, a_bias, decay_scale, key_eps, n, H, D);
    return check_launch("delta_prepare");
}

extern "C" int liyab_delta_scan(float* out, const float* r, const float* k, const float* v, int64_t ld, const float* prep, float* state,
                                int64_t state_stride, int n_slots, const int* seq_starts, const int* positions, const int* state_slots,
                                int n_seqs, int H, int D, hipStream_t stream) {
    LIYAB_REQUIRE(out && r && k && v && prep && state && seq_starts && positions && state_slots, "delta_scan: null pointer");
    LIYAB_REQUIRE(n_seqs >= 0 && H > 0 && liyab_delta_takes(D) && ld >= static_cast<int64_t>(H) * D, "delta_scan: bad sizes H=%d D=%d", H, D);
    LIYAB_REQUIRE(n_slots > 0 && state_stride >= static_cast<int64_t>(H) * D * D, "delta_scan: the slot does not hold the heads' matrices");
    if (n_seqs == 0) return 0;
    DeltaArgs a{out, r, k, v, ld, prep, state, state_stride, n_slots, seq_starts, positions, state_slots, n_seqs, H, D};
    const int64_t items = static_cast<int64_t>(n_seqs) * H * ((D + kDeltaCols - 1) / kDeltaCols);
    const dim3 grid(static_cast<unsigned>((items + kDeltaWaves - 1) / kDeltaWaves));
    const int per = (D + kDeltaSplit - 1) / kDeltaSplit;
    if (per <= 8) delta_scan_kernel<8, true><<<grid, kDeltaWaves * kWave, 0, stream>>>(a);
    else if (per <= 16) delta_scan_kernel<16, true><<<grid, kDeltaWaves * kWave, 0, stream>>>(a);
    else if (per <= 32) delta_scan_kernel<32, false><<<grid, kDeltaWaves * kWave, 0, stream>>>(a);
    else delta_scan_kernel<64, false><<<grid, kDeltaWaves * kWave, 0, stream>>>(a);
    return check_launch("delta_scan");
}

extern "C" int liyab_head_norm_gate(void* out, int out_dtype, const float* o, const float* gate, int64_t ldg, const float* w, float eps, int n,
                                    int H, int D, hipStream_t stream) {
    LIYAB_REQUIRE(out && o, "head_norm_gate: null pointer");
    LIYAB_REQUIRE(n >= 0 && H > 0 && D > 0 && (gate == nullptr || ldg >= static_cast<int64_t>(H) * D), "head_norm_gate: bad sizes");
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "head_norm_gate: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(n) * H + 3) / 4);
    if (out_dtype == kF32) head_norm_gate_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), o, gate, ldg, w, eps, n, H, D);
    else head_norm_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), o, gate, ldg, w, eps, n, H, D);
    return check_launch("head_norm_gate");
}
