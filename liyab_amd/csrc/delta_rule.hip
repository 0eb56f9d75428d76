// A recurrence that decays a head's matrix of state and takes out of it what the token's key already holds there, before the
// token's own outer product is added (a delta rule with a decay and a removal rate a channel):
//   u = k / sqrt(sum(k^2) + key_eps),   w = exp(-decay_scale * sigmoid(wraw + w0)),   a = sigmoid(araw + a_bias)
//   S <- diag(w) S - (a * u)(u^T S) + k v^T         (both terms read the old S; S is [key channel, value channel])
//   o = S^T r
// The map S -> diag(w) S - (a * u)(u^T S) acts on every column of S on its own, so columns never exchange anything.
//
// liyab_delta_prepare: (w, a * u, u) of every token, head and key channel, float32 [n, 3, H * D]: a wave a (token, head).
// liyab_delta_scan: a workgroup a (request, head) (four waves, a block of 16 columns each; heads wider than 64 take several
//   workgroups) walks the request's rows of the step in order. Four lanes side by side share a column, each with a quarter
//   of its rows in registers, so the two sums over the rows of a column (u^T S and S^T r) are sums over a quad of lanes,
//   which come through the lanes' own data path. The tokens' vectors go through LDS a chunk of up to 16 tokens at a time
//   (one trip to memory a chunk, not a token), the next chunk fetched into registers while this one is computed. The state
//   is 32-bit in the request's slot and in registers; it is zero at position 0 whatever the slot holds.
//   A step with long portions (seg_tokens > 0) runs in segments of that many tokens side by side, in three launches. The
//   recurrence is linear in S, S_t = A_t S_(t-1) + k_t v_t^T with A_t = diag(w_t) - (a_t * u_t) u_t^T, so a segment's end is
//   P S_start + Z: every segment but a request's last walks twice side by side, from a zero state for Z and, without the outer
//   products, from the unit matrix for P (the product of its A_t); delta_combine_kernel strings a request's segments together
//   and leaves each the state it starts from; then every segment walks from that state and writes its outputs.
// liyab_head_norm_gate: out = o / sqrt(mean(o^2 over the head) + eps) * weight * sigmoid(gate), rounded once.
// liyab_delta_single: all three for a step of single tokens and heads of up to 64, in one kernel.
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
    // long portions in segments (seg_tokens > 0): a workgroup a (segment, head, ...) instead of a (request, head, ...)
    int seg_tokens, max_segs, phase;  // phase 0: the whole portion in one walk; 1: each segment for Z and P; 3: each segment from its true start
    float* seg_state;         // [segments][H][D][D]: a segment's Z
    float* seg_trans;         // [segments][H][D][D]: a segment's P
    float* seg_start;         // [segments][H][D][D]: the state a segment starts from (the combining pass writes it)
};

// segment `g` of the step in the order of the requests: its request and rows; false past the last segment
__device__ __forceinline__ bool delta_segment(const DeltaArgs& a, int g, int& s, int& begin, int& end, bool& last) {
    for (s = 0; s < a.n_seqs; ++s) {
        const int b = a.seq_starts[s], len = a.seq_starts[s + 1] - b;
        const int n_seg = (len + a.seg_tokens - 1) / a.seg_tokens;
        if (g < n_seg) {
            begin = b + g * a.seg_tokens;
            end = min(begin + a.seg_tokens, b + len);
            last = g == n_seg - 1;
            return true;
        }
        g -= n_seg;
    }
    return false;
}

// REG: rows a lane holds (D <= 4 * REG); a lane's rows are i0 .. i0 + REG - 1, i0 = (lane % 4) * REG. The waves of a workgroup
// are column blocks of one (request, head) and share its tokens' vectors: CH tokens at a time go through LDS (w, a * u, u, k, r
// padded to DP = 4 * REG entries, v), the next CH fetched into registers while these are computed.
// OUT: outputs are written (not in the pass that only wants the segments' ends)
template <int REG, bool OUT>
__global__ void __launch_bounds__(kDeltaWaves * kWave)
delta_scan_kernel(DeltaArgs a) {
    constexpr int DP = 4 * REG;
    constexpr int CH = DP >= 64 ? 1024 / DP : 16;   // tokens a chunk: 16, 16, 8, 4 for REG = 8, 16, 32, 64
    constexpr int PER = 6 * CH * DP;                 // floats a chunk
    constexpr int NPRE = PER / (kDeltaWaves * kWave);
    static_assert(PER % (kDeltaWaves * kWave) == 0, "a chunk is dealt evenly among the threads");
    __shared__ __attribute__((aligned(16))) float lds[2 * PER];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int D = a.D;
    const int n_cb = (D + kDeltaCols - 1) / kDeltaCols;
    const int n_grp = (n_cb + kDeltaWaves - 1) / kDeltaWaves;
    // in phase 1 two workgroups side by side a (segment, head, group of columns): one for Z, one for P
    const int n_kind = a.phase == 1 ? 2 : 1;
    const int kind = blockIdx.x % n_kind, rest = blockIdx.x / n_kind;
    const int grp = rest % n_grp, h = (rest / n_grp) % a.H, item = rest / (n_grp * a.H);
    int s = item, begin, end;
    bool last_seg = true;
    if (a.seg_tokens > 0) {
        if (!delta_segment(a, item, s, begin, end, last_seg)) return;
        if (a.phase == 1 && last_seg) return;  // (nobody needs the end of a request's last segment from zero)
    } else {
        begin = a.seq_starts[s];
        end = a.seq_starts[s + 1];
    }
    if (begin >= end) return;
    const bool homogeneous = kind == 1;  // the walk for P: no outer products, from the unit matrix
    const int cb = grp * kDeltaWaves + wave;
    const int rb = lane % kDeltaSplit, j = cb * kDeltaCols + lane / kDeltaSplit;
    const int i0 = rb * REG;
    const int slot = a.state_slots[s];
    const bool slot_ok = slot >= 0 && slot < a.n_slots;
    const bool fresh = a.positions[begin] == 0;
    float* Sg = a.state + static_cast<int64_t>(slot_ok ? slot : 0) * a.state_stride + static_cast<int64_t>(h) * D * D;
    const int64_t seg_at = (static_cast<int64_t>(item) * a.H + h) * D * D;
    float* S_seg = (a.phase == 3 ? a.seg_start : homogeneous ? a.seg_trans : a.seg_state) + seg_at;  // (written in phase 1, read in phase 3)
    float S[REG];
    bool mine[REG];
#pragma unroll
    for (int ii = 0; ii < REG; ++ii) {
        mine[ii] = i0 + ii < D && j < D;
        if (a.phase == 0) S[ii] = (mine[ii] && slot_ok && !fresh) ? Sg[static_cast<int64_t>(i0 + ii) * D + j] : 0.0f;
        else if (a.phase == 3) S[ii] = mine[ii] ? S_seg[static_cast<int64_t>(i0 + ii) * D + j] : 0.0f;
        else S[ii] = (mine[ii] && homogeneous && i0 + ii == j) ? 1.0f : 0.0f;
    }
    const int64_t HD = static_cast<int64_t>(a.H) * D;
    // element e of a chunk: array e / (CH * DP) (w, a u, u, k, r, v), token (e / DP) % CH, entry e % DP
    float pre[NPRE];
    auto fetch = [&](int c0) {
#pragma unroll
        for (int q = 0; q < NPRE; ++q) {
            const int e = tid + q * (kDeltaWaves * kWave);
            const int arr = e / (CH * DP), tt = (e / DP) % CH, i = e % DP;
            const int t = min(c0 + tt, end - 1), ic = min(i, D - 1);
            const float* src = arr < 3 ? a.prep + static_cast<int64_t>(t) * 3 * HD + arr * HD + h * D + ic
                                       : (arr == 3 ? a.k : arr == 4 ? a.r : a.v) + static_cast<int64_t>(t) * a.ld + h * D + ic;
            const float val = *src;
            pre[q] = i < D ? val : 0.0f;
        }
    };
    auto stash = [&](float* buf) {
#pragma unroll
        for (int q = 0; q < NPRE; ++q) buf[tid + q * (kDeltaWaves * kWave)] = pre[q];
    };
    fetch(begin);
    stash(lds);
    __syncthreads();
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    int which = 0;
    for (int c0 = begin; c0 < end; c0 += CH) {
        const bool more = c0 + CH < end;
        if (more) fetch(c0 + CH);
        const float* buf = lds + which * PER;
        const int n_tok = min(CH, end - c0);
        for (int tt = 0; tt < n_tok; ++tt) {
            const float* w = buf + tt * DP + i0;
            const float* au = w + CH * DP;
            const float* u = au + CH * DP;
            const float* k = u + CH * DP;
            const float* r = k + CH * DP;
            const float v = homogeneous ? 0.0f : buf[5 * CH * DP + tt * DP + min(j, DP - 1)];
            // four sums side by side (one a place of a piece of four rows), added at the end: a chain a quarter as long
            f32x4 seen4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int q4 = 0; q4 < REG / 4; ++q4) {
                const f32x4 u4 = *reinterpret_cast<const f32x4*>(u + 4 * q4);
#pragma unroll
                for (int e = 0; e < 4; ++e) seen4[e] += u4[e] * S[4 * q4 + e];   // (rows that are not this lane's hold zero)
            }
            const float seen = group_sum<kDeltaSplit>((seen4[0] + seen4[1]) + (seen4[2] + seen4[3]));
            f32x4 o4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int q4 = 0; q4 < REG / 4; ++q4) {
                const f32x4 w4 = *reinterpret_cast<const f32x4*>(w + 4 * q4), a4 = *reinterpret_cast<const f32x4*>(au + 4 * q4);
                const f32x4 k4 = *reinterpret_cast<const f32x4*>(k + 4 * q4), r4 = *reinterpret_cast<const f32x4*>(r + 4 * q4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int ii = 4 * q4 + e;
                    S[ii] = mine[ii] ? w4[e] * S[ii] - a4[e] * seen + k4[e] * v : 0.0f;
                    if (OUT) o4[e] += r4[e] * S[ii];
                }
            }
            if (OUT) {
                float o = (o4[0] + o4[1]) + (o4[2] + o4[3]);
                o = group_sum<kDeltaSplit>(o);
                if (rb == 0 && j < D) a.out[static_cast<int64_t>(c0 + tt) * HD + h * D + j] = o;
            }
        }
        if (more) stash(lds + (which ^ 1) * PER);
        __syncthreads();
        which ^= 1;
    }
    if (a.phase == 1) {
#pragma unroll
        for (int ii = 0; ii < REG; ++ii)
            if (mine[ii]) S_seg[static_cast<int64_t>(i0 + ii) * D + j] = S[ii];
    } else if (slot_ok && last_seg) {
#pragma unroll
        for (int ii = 0; ii < REG; ++ii)
            if (mine[ii]) Sg[static_cast<int64_t>(i0 + ii) * D + j] = S[ii];
    }
}

// Between the two passes over the segments: the state each segment starts from. A workgroup a (request, head, block of 16
// columns) walks the request's segments in order, S <- P S + Z, and leaves in seg_start what each segment starts from (the
// first: the slot's state, or zeros at position 0); an array of its own, named as such to the compiler, so that no load of a
// later segment's Z or P has to wait behind a store. A thread holds rows ib, ib + 16, ... of one column; the columns' block
// of S lies in LDS; P goes through LDS in tiles of 64 x 64, the next tile fetched into registers while this one is used.
constexpr int kCombTile = 64, kCombStride = kCombTile + 4;  // (rows 68 floats apart: four rows read together fall into different banks)
constexpr int kCombMaxD = 256;

__global__ void __launch_bounds__(256)
delta_combine_kernel(DeltaArgs a, const float* __restrict__ seg_z, const float* __restrict__ seg_p, float* __restrict__ seg_start) {
    __shared__ __attribute__((aligned(16))) float Pt[kCombTile * kCombStride];
    __shared__ float Sl[2][kCombMaxD * kDeltaCols];
    const int s = blockIdx.x, h = blockIdx.y, cb = blockIdx.z, tid = threadIdx.x;
    const int D = a.D, H = a.H;
    int g0 = 0;
    for (int q = 0; q < s; ++q) g0 += (a.seq_starts[q + 1] - a.seq_starts[q] + a.seg_tokens - 1) / a.seg_tokens;
    const int begin = a.seq_starts[s];
    const int n_seg = (a.seq_starts[s + 1] - begin + a.seg_tokens - 1) / a.seg_tokens;
    if (n_seg <= 0) return;
    const int slot = a.state_slots[s];
    const bool from_slot = slot >= 0 && slot < a.n_slots && a.positions[begin] != 0;
    const int jj = tid % kDeltaCols, ib = tid / kDeltaCols, j = cb * kDeltaCols + jj;
    const int64_t DD = static_cast<int64_t>(D) * D;
    const float* S0 = a.state + static_cast<int64_t>(from_slot ? slot : 0) * a.state_stride + h * DD;
    for (int m = ib; m < kCombMaxD; m += 256 / kDeltaCols) {  // (rows past the head's last stay zero: they meet zeros of P)
        Sl[0][m * kDeltaCols + jj] = (from_slot && m < D && j < D) ? S0[static_cast<int64_t>(m) * D + j] : 0.0f;
        Sl[1][m * kDeltaCols + jj] = 0.0f;
    }
    const int nb = (D + kCombTile - 1) / kCombTile, per_seg = nb * nb;
    const int n_tiles = (n_seg - 1) * per_seg;
    constexpr int NPRE = kCombTile * kCombTile / 256;
    float pre[NPRE];
    auto fetch = [&](int T) {
        const int g = T / per_seg, ibk = (T % per_seg) / nb, mbk = T % nb;
        const float* P = seg_p + (static_cast<int64_t>(g0 + g) * H + h) * DD;
#pragma unroll
        for (int q = 0; q < NPRE; ++q) {
            const int e = tid + q * 256;
            const int i = ibk * kCombTile + e / kCombTile, m = mbk * kCombTile + e % kCombTile;
            const float val = P[static_cast<int64_t>(min(i, D - 1)) * D + min(m, D - 1)];
            pre[q] = (i < D && m < D) ? val : 0.0f;
        }
    };
    // a segment's own end, for the rows of block ibk of step g * nb + ibk; asked for one step ahead, like the tiles (the barriers
    // below wait for LDS only, so what is on its way from memory stays on its way)
    auto fetch_z = [&](int step, float (&z)[4]) {
        const int g = step / nb, ibk = step % nb;
        const bool live = g + 1 < n_seg;  // (a request's last segment has none)
        const float* Zg = seg_z + (static_cast<int64_t>(g0 + g) * H + h) * DD;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int i = ibk * kCombTile + ib + 16 * q;
            z[q] = (live && i < D && j < D) ? Zg[static_cast<int64_t>(i) * D + j] : 0.0f;
        }
    };
    float z_next[4];
    fetch_z(0, z_next);
    if (n_tiles > 0) fetch(0);
    __syncthreads();
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    int cur = 0;
    for (int g = 0; g < n_seg; ++g) {
        float* Sg = seg_start + (static_cast<int64_t>(g0 + g) * H + h) * DD;
        const bool more = g + 1 < n_seg;
        for (int ibk = 0; ibk < nb; ++ibk) {
            float acc[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] = z_next[q];
            if (g * nb + ibk + 1 < n_seg * nb) fetch_z(g * nb + ibk + 1, z_next);
            if (more) {
                for (int mbk = 0; mbk < nb; ++mbk) {
                    const int T = (g * nb + ibk) * nb + mbk;
#pragma unroll
                    for (int q = 0; q < NPRE; ++q) {
                        const int e = tid + q * 256;
                        Pt[(e / kCombTile) * kCombStride + e % kCombTile] = pre[q];
                    }
                    lds_barrier();
                    if (T + 1 < n_tiles) fetch(T + 1);
                    const float* Sc = Sl[cur] + mbk * kCombTile * kDeltaCols + jj;
#pragma unroll 4
                    for (int c = 0; c < kCombTile; c += 4) {
                        float sv[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) sv[e] = Sc[(c + e) * kDeltaCols];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const f32x4 p4 = *reinterpret_cast<const f32x4*>(Pt + (ib + 16 * q) * kCombStride + c);
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[q] += p4[e] * sv[e];
                        }
                    }
                    lds_barrier();  // (the next tile takes this one's place)
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int i = ibk * kCombTile + ib + 16 * q;
                if (i < D) Sl[cur ^ 1][i * kDeltaCols + jj] = acc[q];
            }
        }
        if (j < D)
            for (int m = ib; m < D; m += 256 / kDeltaCols) Sg[static_cast<int64_t>(m) * D + j] = Sl[cur][m * kDeltaCols + jj];
        lds_barrier();
        cur ^= 1;
    }
}

// A step in which every request brings one token, heads of up to 64: what liyab_delta_prepare, liyab_delta_scan and
// liyab_head_norm_gate do in turn, in one kernel, a workgroup a (request, head). The first wave takes the token's decays, rates
// and unit key and leaves the six vectors in LDS, every wave walks its block of columns for this one token, and the first wave
// norms and gates the head's result. The arithmetic and its order are those of the three kernels (the same bits).
struct DeltaSingleArgs {
    void* out;                // [n, H * D], the compute type
    const float *r, *k, *v, *araw, *gate;  // rows of ld floats, a head's D values at h * D
    int64_t ld;
    const float* wraw;        // rows of ldw floats
    int64_t ldw;
    const float *w0, *a_bias, *norm_w;
    float eps, decay_scale, key_eps;
    float* state;
    int64_t state_stride;
    int n_slots;
    const int* seq_starts;
    const int* positions;
    const int* state_slots;
    int n_seqs, H, D;
};

template <typename T, int REG>
__global__ void __launch_bounds__(kDeltaWaves * kWave)
delta_single_kernel(DeltaSingleArgs a) {
    constexpr int DP = 4 * REG;  // 32 or 64
    static_assert(DP <= kWave, "the first wave holds a head's vectors, an entry a lane");
    __shared__ __attribute__((aligned(16))) float vec[6 * DP];  // w, a * u, u, k, r, v
    __shared__ float o_s[kDeltaWaves * kDeltaCols];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int h = blockIdx.x % a.H, s = blockIdx.x / a.H;
    const int t = a.seq_starts[s];
    if (a.seq_starts[s + 1] - t != 1) return;  // (the host sends steps of single tokens only)
    const int D = a.D;
    if (wave == 0) {
        const bool in = lane < D;
        const int64_t at = static_cast<int64_t>(t) * a.ld + h * D + (in ? lane : 0);
        const int ch = h * D + (in ? lane : 0);
        const float k = in ? a.k[at] : 0.0f, r = in ? a.r[at] : 0.0f, v = in ? a.v[at] : 0.0f;
        const float inv = 1.0f / sqrtf(wave_sum(k * k) + a.key_eps);
        const float u = k * inv;
        const float w = expf(-a.decay_scale * sigmoid_f(a.wraw[static_cast<int64_t>(t) * a.ldw + ch] + a.w0[ch]));
        const float rate = sigmoid_f(a.araw[at] + a.a_bias[ch]);
        if (lane < DP) {
            vec[lane] = in ? w : 0.0f;
            vec[DP + lane] = in ? rate * u : 0.0f;
            vec[2 * DP + lane] = u;
            vec[3 * DP + lane] = k;
            vec[4 * DP + lane] = r;
            vec[5 * DP + lane] = v;
        }
    }
    __syncthreads();
    const int rb = lane % kDeltaSplit, j = wave * kDeltaCols + lane / kDeltaSplit;
    const int i0 = rb * REG;
    const int slot = a.state_slots[s];
    const bool slot_ok = slot >= 0 && slot < a.n_slots;
    const bool fresh = a.positions[t] == 0;
    float* Sg = a.state + static_cast<int64_t>(slot_ok ? slot : 0) * a.state_stride + static_cast<int64_t>(h) * D * D;
    float S[REG];
    bool mine[REG];
#pragma unroll
    for (int ii = 0; ii < REG; ++ii) {
        mine[ii] = i0 + ii < D && j < D;
        S[ii] = (mine[ii] && slot_ok && !fresh) ? Sg[static_cast<int64_t>(i0 + ii) * D + j] : 0.0f;
    }
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    const float* w = vec + i0;
    const float* au = w + DP;
    const float* u = au + DP;
    const float* k = u + DP;
    const float* r = k + DP;
    const float v = vec[5 * DP + min(j, DP - 1)];
    f32x4 seen4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q4 = 0; q4 < REG / 4; ++q4) {
        const f32x4 u4 = *reinterpret_cast<const f32x4*>(u + 4 * q4);
#pragma unroll
        for (int e = 0; e < 4; ++e) seen4[e] += u4[e] * S[4 * q4 + e];
    }
    const float seen = group_sum<kDeltaSplit>((seen4[0] + seen4[1]) + (seen4[2] + seen4[3]));
    f32x4 o4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q4 = 0; q4 < REG / 4; ++q4) {
        const f32x4 w4 = *reinterpret_cast<const f32x4*>(w + 4 * q4), a4 = *reinterpret_cast<const f32x4*>(au + 4 * q4);
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(k + 4 * q4), r4 = *reinterpret_cast<const f32x4*>(r + 4 * q4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int ii = 4 * q4 + e;
            S[ii] = mine[ii] ? w4[e] * S[ii] - a4[e] * seen + k4[e] * v : 0.0f;
            o4[e] += r4[e] * S[ii];
        }
    }
    const float o = group_sum<kDeltaSplit>((o4[0] + o4[1]) + (o4[2] + o4[3]));
    if (rb == 0) o_s[j] = j < D ? o : 0.0f;
    if (slot_ok) {
#pragma unroll
        for (int ii = 0; ii < REG; ++ii)
            if (mine[ii]) Sg[static_cast<int64_t>(i0 + ii) * D + j] = S[ii];
    }
    __syncthreads();
    if (wave == 0) {
        const bool in = lane < D;
        const float ov = in ? o_s[lane] : 0.0f;
        const float scale = 1.0f / sqrtf(wave_sum(ov * ov) / static_cast<float>(D) + a.eps);
        if (in) {
            float y = ov * scale;
            if (a.norm_w != nullptr) y *= a.norm_w[h * D + lane];
            if (a.gate != nullptr) y *= sigmoid_f(a.gate[static_cast<int64_t>(t) * a.ld + h * D + lane]);
            static_cast<T*>(a.out)[(static_cast<int64_t>(t) * a.H + h) * D + lane] = from_float<T>(y);
        }
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
                                int n_seqs, int H, int D, int seg_tokens, int max_segs, float* seg_state, float* seg_trans, float* seg_start,
                                hipStream_t stream) {
    LIYAB_REQUIRE(out && r && k && v && prep && state && seq_starts && positions && state_slots, "delta_scan: null pointer");
    LIYAB_REQUIRE(seg_tokens >= 0 && (seg_tokens == 0 || (max_segs > 0 && seg_state && seg_trans && seg_start)), "delta_scan: segments need their count and scratch");
    LIYAB_REQUIRE(n_seqs >= 0 && H > 0 && liyab_delta_takes(D) && ld >= static_cast<int64_t>(H) * D, "delta_scan: bad sizes H=%d D=%d", H, D);
    LIYAB_REQUIRE(n_slots > 0 && state_stride >= static_cast<int64_t>(H) * D * D, "delta_scan: the slot does not hold the heads' matrices");
    if (n_seqs == 0) return 0;
    DeltaArgs a{out, r, k, v, ld, prep, state, state_stride, n_slots, seq_starts, positions, state_slots, n_seqs, H, D,
                seg_tokens, max_segs, 0, seg_state, seg_trans, seg_start};
    const int n_cb = (D + kDeltaCols - 1) / kDeltaCols;
    const int per = (D + kDeltaSplit - 1) / kDeltaSplit;
    const int64_t per_item = static_cast<int64_t>(H) * ((n_cb + kDeltaWaves - 1) / kDeltaWaves);
    auto walk = [&](const DeltaArgs& p, int64_t items, bool outputs) {
        const dim3 grid(static_cast<unsigned>(items * per_item));
        constexpr int T = kDeltaWaves * kWave;
        if (outputs) {
            if (per <= 8) delta_scan_kernel<8, true><<<grid, T, 0, stream>>>(p);
            else if (per <= 16) delta_scan_kernel<16, true><<<grid, T, 0, stream>>>(p);
            else if (per <= 32) delta_scan_kernel<32, true><<<grid, T, 0, stream>>>(p);
            else delta_scan_kernel<64, true><<<grid, T, 0, stream>>>(p);
        } else {
            if (per <= 8) delta_scan_kernel<8, false><<<grid, T, 0, stream>>>(p);
            else if (per <= 16) delta_scan_kernel<16, false><<<grid, T, 0, stream>>>(p);
            else if (per <= 32) delta_scan_kernel<32, false><<<grid, T, 0, stream>>>(p);
            else delta_scan_kernel<64, false><<<grid, T, 0, stream>>>(p);
        }
    };
    if (seg_tokens > 0) {
        // segments side by side: each for its end from zero and its transition, the ends strung together, each again from its true start
        DeltaArgs p = a;
        p.phase = 1;
        walk(p, static_cast<int64_t>(max_segs) * 2, false);
        delta_combine_kernel<<<dim3(n_seqs, H, n_cb), 256, 0, stream>>>(p, seg_state, seg_trans, seg_start);
        p.phase = 3;
        walk(p, max_segs, true);
        return check_launch("delta_scan");
    }
    walk(a, n_seqs, true);
    return check_launch("delta_scan");
}

extern "C" int liyab_delta_single_takes(int D) { return D >= 1 && D <= 64 ? 1 : 0; }

extern "C" int liyab_delta_single(void* out, int out_dtype, const float* r, const float* k, const float* v, const float* araw, const float* gate,
                                  int64_t ld, const float* wraw, int64_t ldw, const float* w0, const float* a_bias, const float* norm_w, float eps,
                                  float decay_scale, float key_eps, float* state, int64_t state_stride, int n_slots, const int* seq_starts,
                                  const int* positions, const int* state_slots, int n_seqs, int H, int D, hipStream_t stream) {
    LIYAB_REQUIRE(out && r && k && v && araw && wraw && w0 && a_bias && state && seq_starts && positions && state_slots, "delta_single: null pointer");
    LIYAB_REQUIRE(n_seqs >= 0 && H > 0 && liyab_delta_single_takes(D) && ld >= static_cast<int64_t>(H) * D && ldw >= static_cast<int64_t>(H) * D,
                  "delta_single: bad sizes H=%d D=%d", H, D);
    LIYAB_REQUIRE(n_slots > 0 && state_stride >= static_cast<int64_t>(H) * D * D, "delta_single: the slot does not hold the heads' matrices");
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "delta_single: unknown dtype %d", out_dtype);
    if (n_seqs == 0) return 0;
    DeltaSingleArgs a{out, r, k, v, araw, gate, ld, wraw, ldw, w0, a_bias, norm_w, eps, decay_scale, key_eps, state, state_stride, n_slots,
                      seq_starts, positions, state_slots, n_seqs, H, D};
    const dim3 grid(static_cast<unsigned>(static_cast<int64_t>(n_seqs) * H));
    constexpr int T = kDeltaWaves * kWave;
    if (out_dtype == kF32) {
        if (D <= 32) delta_single_kernel<float, 8><<<grid, T, 0, stream>>>(a);
        else delta_single_kernel<float, 16><<<grid, T, 0, stream>>>(a);
    } else {
        if (D <= 32) delta_single_kernel<bf16_t, 8><<<grid, T, 0, stream>>>(a);
        else delta_single_kernel<bf16_t, 16><<<grid, T, 0, stream>>>(a);
    }
    return check_launch("delta_single");
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
